"""Python faces of the HIP launchers: they take torch tensors (used purely as
device allocations), check dtypes and contiguity, and pass raw pointers and
the current HIP stream to libshrike_hip.  Nothing here computes anything."""

from __future__ import annotations

import torch

from .lib import KernelError, check, load

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _CODES[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16 tensors, got {dtype}") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_device_index: int | None = None


def _stream() -> int:
    """Handle of the current HIP stream (the capture stream while a graph is recorded).
    The engine runs on one GPU: its index is asked for once."""
    global _device_index
    if _device_index is None:
        _device_index = torch.cuda.current_device()
    if _raw_stream is not None:  # a tenth of the cost of building a torch.cuda.Stream object
        return _raw_stream(_device_index)
    return torch.cuda.current_stream().cuda_stream


def current_stream() -> int:
    """Handle of the HIP stream that launches go to now."""
    return _stream()


def _dev(t: torch.Tensor, name: str, dtype=None) -> int:
    if not t.is_cuda:
        raise KernelError(f"{name}: expected a device tensor (there is no CPU path)")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: expected {dtype}, got {t.dtype}")
    return t.data_ptr()


def _rows(t: torch.Tensor, name: str) -> None:
    if t.dim() != 2 or t.stride(1) != 1:
        raise KernelError(f"{name}: expected a 2-d tensor with unit inner stride")


class SplitSum:
    """The float32 partial sums [splits, n, m] of a product that was split
    along k, with the bias that is still to be added.  Kernels that read the
    product (add_rmsnorm, rope_kv_store) add the parts up in order."""

    __slots__ = ("parts", "bias")

    def __init__(self, parts: torch.Tensor, bias: torch.Tensor | None = None):
        self.parts = parts
        self.bias = bias

    @property
    def shape(self):
        return self.parts.shape[1:]


def _words(t: torch.Tensor, name: str) -> int:
    """Address of an int32 tensor that a kernel may touch: on the device, or page-locked."""
    if t.dtype != torch.int32 or not t.is_contiguous() or not (t.is_cuda or t.is_pinned()):
        raise KernelError(f"{name}: expected a contiguous int32 tensor on the device or in page-locked memory")
    return t.data_ptr()


def copy_words(src: torch.Tensor, dst: torch.Tensor, patch: torch.Tensor | None = None, patch_at: int = 0) -> None:
    """dst[:] = src[:] (int32, equal lengths) by a kernel, with dst[patch_at : patch_at +
    len(patch)] taken from `patch` instead.  Either tensor may be page-locked host memory."""
    n = src.numel()
    if dst.numel() != n:
        raise KernelError("copy_words: src and dst differ in length")
    patch_n = 0 if patch is None else patch.numel()
    if patch_at < 0 or patch_at + patch_n > n:
        raise KernelError("copy_words: the patch does not fit")
    check(load().shk_copy_words(_words(src, "src"), _words(dst, "dst"), n,
                                None if patch is None else _words(patch, "patch"), patch_at, patch_n, _stream()))


def gather_rows(src: torch.Tensor, index: torch.Tensor, dst: torch.Tensor) -> None:
    """dst[r] = src[index[r]] for 2-d tensors of a 4-byte dtype (src rows may be
    strided); index int32, on the device or page-locked, every entry below src's
    row count (the caller's promise: nothing on the device checks it)."""
    _rows(src, "gather_rows src")
    if (dst.dim() != 2 or not dst.is_contiguous() or dst.dtype != src.dtype or src.element_size() != 4
            or dst.shape[1] != src.shape[1] or index.numel() != dst.shape[0]):
        raise KernelError("gather_rows: dst must be contiguous [len(index), width] of src's 4-byte dtype")
    check(load().shk_gather_rows(_dev(src, "src"), src.stride(0), src.shape[0], _words(index, "index"),
                                 _dev(dst, "dst"), dst.shape[0], dst.shape[1], _stream()))


def zero_(t: torch.Tensor) -> None:
    """Fills a contiguous device tensor with zero bytes by a kernel of the library."""
    if not t.is_contiguous():
        raise KernelError("zero_: expected a contiguous tensor")
    check(load().shk_zero_bytes(_dev(t, "t"), t.numel() * t.element_size(), _stream()))


def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
    """out[i] = float(table[ids[i]]); ids int32 [n], out float32 [n, hidden]."""
    n, hidden = out.shape
    if not (table.is_contiguous() and out.is_contiguous() and table.shape[1] == hidden):
        raise KernelError("embed: table/out must be contiguous with the same width")
    check(
        load().shk_embed(
            _dev(table, "table"), dtype_code(table.dtype), _dev(ids, "ids", torch.int32),
            _dev(out, "out", torch.float32), n, hidden, table.shape[0], _stream(),
        )
    )


def add_rmsnorm(resid, delta, weight, eps: float, out, rows=None, write_resid=True) -> None:
    """resid (+= delta); out = rmsnorm(resid) * weight.  With `rows` (int32 [n])
    only those rows are normed, into out[0..n)."""
    n, hidden = out.shape
    if not (resid.is_contiguous() and out.is_contiguous() and resid.shape[1] == hidden):
        raise KernelError("add_rmsnorm: resid/out must be contiguous with the same width")
    splits = 0
    if isinstance(delta, SplitSum):
        if delta.bias is not None or tuple(delta.shape) != tuple(resid.shape):
            raise KernelError("add_rmsnorm: partial sums must match resid's shape and carry no bias")
        splits, delta = delta.parts.shape[0], delta.parts
        if delta.dtype != torch.float32 or not delta.is_contiguous():
            raise KernelError("add_rmsnorm: partial sums must be contiguous float32")
    elif delta is not None and (
        delta.dtype != out.dtype or not delta.is_contiguous() or delta.shape != resid.shape
    ):
        raise KernelError("add_rmsnorm: delta must match resid's shape and out's dtype")
    if weight.numel() != hidden:
        raise KernelError(f"add_rmsnorm: weight has {weight.numel()} elements, hidden is {hidden}")
    if rows is None and resid.shape[0] != n:
        raise KernelError("add_rmsnorm: out and resid differ in rows")
    check(
        load().shk_add_rmsnorm(
            _dev(resid, "resid", torch.float32),
            None if delta is None else _dev(delta, "delta"),
            _dev(weight, "weight", torch.float32), float(eps), _dev(out, "out"),
            dtype_code(out.dtype), None if rows is None else _dev(rows, "rows", torch.int32),
            n, hidden, int(bool(write_resid)), splits, resid.shape[0], _stream(),
        )
    )


GATE_ACTIVATIONS = {"silu": 1, "gelu_tanh": 2}


def activation_code(gated) -> int:
    """0 for a product that is not gated; else the code of the gate's activation
    (True stands for "silu")."""
    if not gated:
        return 0
    name = "silu" if gated is True else gated
    try:
        return GATE_ACTIVATIONS[name]
    except KeyError:
        raise KernelError(f"gate activation must be one of {sorted(GATE_ACTIVATIONS)}, got {gated!r}") from None


def act_mul(gate_up: torch.Tensor, out: torch.Tensor, activation: str = "silu") -> None:
    """out = act(gate_up[:, :I]) * gate_up[:, I:]."""
    n, inter = out.shape
    if gate_up.shape != (n, 2 * inter) or not gate_up.is_contiguous() or not out.is_contiguous():
        raise KernelError("act_mul: gate_up must be contiguous [n, 2*inter]")
    if gate_up.dtype != out.dtype:
        raise KernelError("act_mul: dtypes differ")
    check(load().shk_act_mul(_dev(gate_up, "gate_up"), _dev(out, "out"), dtype_code(out.dtype),
                             n, inter, activation_code(activation), _stream()))


def gemm(a, w, out, bias=None, accumulate=False) -> None:
    """out (+)= a @ w.T + bias;  a [n, k], w [m, k] contiguous, out [n, m]."""
    _rows(a, "gemm a")
    _rows(out, "gemm out")
    n, k = a.shape
    m = w.shape[0]
    if w.dim() != 2 or w.shape[1] != k or not w.is_contiguous():
        raise KernelError(f"gemm: w must be contiguous [m, {k}], got {tuple(w.shape)}")
    if out.shape != (n, m):
        raise KernelError(f"gemm: out must be [{n}, {m}], got {tuple(out.shape)}")
    if a.dtype != w.dtype:
        raise KernelError(f"gemm: a is {a.dtype} but w is {w.dtype}")
    if bias is not None and bias.numel() != m:
        raise KernelError(f"gemm: bias has {bias.numel()} elements, m is {m}")
    check(
        load().shk_gemm(
            _dev(a, "a"), _dev(w, "w"),
            None if bias is None else _dev(bias, "bias", torch.float32),
            _dev(out, "out"), n, m, k, a.stride(0), out.stride(0),
            dtype_code(a.dtype), dtype_code(out.dtype), int(bool(accumulate)), _stream(),
        )
    )


def tiled_numel(m: int, k: int) -> int:
    """bfloat16 elements of the tiled layout of an [m, k] matrix."""
    return -(-m // 16) * -(-k // 32) * 512


def retile_weight(w: torch.Tensor) -> torch.Tensor:
    """The MFMA operand layout of a row-major bfloat16 [m, k] matrix (a flat tensor)."""
    if w.dim() != 2 or not w.is_contiguous() or w.dtype != torch.bfloat16:
        raise KernelError("retile_weight: expected a contiguous bfloat16 matrix")
    m, k = w.shape
    wt = torch.empty(tiled_numel(m, k), dtype=torch.bfloat16, device=w.device)
    check(load().shk_retile_weight(_dev(w, "w"), m, k, _dev(wt, "wt"), _stream()))
    return wt


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """The tiled layouts of two row-major [m, k] matrices interleaved by blocks of
    16 rows, for the gated product of gemm_tiled_weight."""
    if gate.shape != up.shape:
        raise KernelError("interleave_gate_up: gate and up differ in shape")
    m, k = gate.shape
    gt, ut = retile_weight(gate), retile_weight(up)
    wt = torch.empty(2 * tiled_numel(m, k), dtype=torch.bfloat16, device=gate.device)
    check(load().shk_interleave_gate_up(_dev(gt, "gate"), _dev(ut, "up"), m, k, _dev(wt, "wt"),
                                        _stream()))
    return wt


def gemm_splits(n: int, m: int, k: int) -> int:
    """Shares of k that fill the chip for an [n, k] x [m, k]^T product (1: do not split)."""
    return int(load().shk_gemm_bf16_splits(n, m, k))


def gemm_parts(n: int, m: int, k: int, gated: bool = False) -> int:
    """Launches that an [n, k] x [m, k]^T product is made of (2: rows whose tiles
    fill whole rounds of the compute units, then the rest)."""
    return int(load().shk_gemm_bf16_parts(n, m, k, int(gated)))


def mfma_alone(operands: torch.Tensor, workgroups: int, iters: int) -> float:
    """Runs the bfloat16 matrix instruction by itself on `operands` (at least
    32,768 bfloat16 values, held in registers) and returns the flop it did:
    for measuring what the matrix units give on operands of a given kind."""
    if operands.dtype != torch.bfloat16 or operands.numel() < 32768 or not operands.is_contiguous():
        raise KernelError("mfma_alone: operands must be 32,768 contiguous bfloat16 values or more")
    out = torch.empty(workgroups * 256, dtype=torch.float32, device=operands.device)
    check(load().shk_mfma_alone(_dev(operands, "operands"), _dev(out, "out", torch.float32), workgroups, iters,
                                _stream()))
    return 2.0 * 64 * 64 * 32 * 4 * workgroups * iters


def gemm_tiled_weight(a, wt, m: int, k: int, out, bias=None, accumulate=False, gated=False,
                      splits: int = 1) -> None:
    """out (+)= a @ w.T + bias with wt = retile_weight(w): up to 64 rows of a
    stream the weights once; more rows run the LDS-staged MFMA kernel (tiles of
    128 x 128 to 256 x 256, chosen by how many the product has).
    splits > 1: out is float32 [splits, n, m] and receives partial sums.
    gated: False, or the gate's activation ("silu", "gelu_tanh"; True is "silu") for
    an interleaved gate/up weight."""
    _rows(a, "gemm a")
    n = a.shape[0]
    if a.shape[1] != k or a.dtype != torch.bfloat16:
        raise KernelError(f"gemm_tiled_weight: a must be bfloat16 [n, {k}], got {tuple(a.shape)}")
    if splits > 1:
        if tuple(out.shape) != (splits, n, m) or not out.is_contiguous() or out.dtype != torch.float32:
            raise KernelError(f"gemm_tiled_weight: partial sums must be contiguous float32 [{splits}, {n}, {m}]")
    else:
        _rows(out, "gemm out")
        if out.shape != (n, m):
            raise KernelError(f"gemm_tiled_weight: out must be [{n}, {m}], got {tuple(out.shape)}")
    if wt.numel() != (2 if gated else 1) * tiled_numel(m, k) or wt.dtype != torch.bfloat16:
        raise KernelError("gemm_tiled_weight: wt is not the tiled layout of an [m, k] matrix")
    if bias is not None and bias.numel() != m:
        raise KernelError(f"gemm_tiled_weight: bias has {bias.numel()} elements, m is {m}")
    check(
        load().shk_gemm_bf16_tiled_weight(
            _dev(a, "a"), _dev(wt, "wt"),
            None if bias is None else _dev(bias, "bias", torch.float32),
            _dev(out, "out"), n, m, k, a.stride(0), out.stride(-2), dtype_code(out.dtype),
            int(bool(accumulate)), activation_code(gated), int(splits), _stream(),
        )
    )


def key_slab(head_dim: int) -> int:
    """Elements per slab of the cached keys: 32, or the whole row where head_dim
    is no multiple of 32 (csrc/common.h: key_slab)."""
    return 32 if head_dim % 32 == 0 else head_dim


def key_pool_shape(pages: int, kv_heads: int, page_size: int, head_dim: int) -> tuple:
    """Keys of a page and head lie in slabs: [pages, kv_heads, head_dim / slab, page_size, slab]."""
    slab = key_slab(head_dim)
    return (pages, kv_heads, head_dim // slab, page_size, slab)


def _check_pools(who, q, tables, k_pool, v_pool, kv_heads, head_dim, page_size) -> None:
    """Keys in slabs (key_pool_shape); values transposed [pages, kv_heads, head_dim, page_size]."""
    pages = k_pool.shape[0]
    if tuple(k_pool.shape) != key_pool_shape(pages, kv_heads, page_size, head_dim):
        raise KernelError(f"{who}: key pool must be {list(key_pool_shape('pages', kv_heads, page_size, head_dim))}, "
                          f"got {tuple(k_pool.shape)}")
    if tuple(v_pool.shape) != (pages, kv_heads, head_dim, page_size):
        raise KernelError(f"{who}: value pool must be [pages, {kv_heads}, {head_dim}, {page_size}], "
                          f"got {tuple(v_pool.shape)}")
    if k_pool.dtype != q.dtype or v_pool.dtype != q.dtype:
        raise KernelError(f"{who}: pools and queries differ in dtype")
    if not (k_pool.is_contiguous() and v_pool.is_contiguous() and tables.is_contiguous()):
        raise KernelError(f"{who}: pools and tables must be contiguous")
    if tables.dim() != 2:
        raise KernelError(f"{who}: tables must be [sequences, blocks]")


def rope_kv_store(qkv, heads, kv_heads, head_dim, rot_dim, inv_freq, positions, token_seq,
                  tables, k_pool, v_pool, page_size, write_kv=True, split_sum=None) -> None:
    """Rotate q and k of qkv [n, (heads + 2 kv_heads) head_dim] in float32 and put
    k, v into their pages (keys in slabs, see key_pool_shape; values transposed
    [pages, kv_heads, head_dim, page_size])."""
    n = qkv.shape[0]
    if not qkv.is_contiguous() or qkv.shape[1] != (heads + 2 * kv_heads) * head_dim:
        raise KernelError("rope_kv_store: qkv must be contiguous [n, (heads + 2 kv_heads) head_dim]")
    # the kernel reads one position (and one sequence index) per row of qkv
    if positions.shape[0] < n or (write_kv and token_seq.shape[0] < n):
        raise KernelError(f"rope_kv_store: qkv has {n} rows but positions / token_seq are shorter")
    parts, splits, bias = None, 0, None
    if split_sum is not None:
        parts, bias = split_sum.parts, split_sum.bias
        splits = parts.shape[0]
        if tuple(parts.shape[1:]) != tuple(qkv.shape) or parts.dtype != torch.float32 or not parts.is_contiguous():
            raise KernelError("rope_kv_store: partial sums must be contiguous float32 [splits, n, width]")
    num_pages = 0
    if write_kv:
        _check_pools("rope_kv_store", qkv, tables, k_pool, v_pool, kv_heads, head_dim, page_size)
        num_pages = k_pool.shape[0]
    check(
        load().shk_rope_kv_store(
            _dev(qkv, "qkv"), dtype_code(qkv.dtype), n, heads, kv_heads, head_dim, rot_dim,
            None if inv_freq is None else _dev(inv_freq, "inv_freq", torch.float32),
            _dev(positions, "positions", torch.int32),
            _dev(token_seq, "token_seq", torch.int32) if write_kv else None,
            _dev(tables, "tables", torch.int32) if write_kv else None,
            tables.shape[1] if write_kv else 0,
            _dev(k_pool, "k_pool") if write_kv else None,
            _dev(v_pool, "v_pool") if write_kv else None,
            page_size, num_pages, int(bool(write_kv)),
            None if parts is None else _dev(parts, "parts", torch.float32), splits,
            None if bias is None else _dev(bias, "bias", torch.float32), _stream(),
        )
    )


def attention(q, out, heads, kv_heads, head_dim, positions, token_seq, tables, k_pool, v_pool,
              page_size, window, scale) -> None:
    """q: [n, >= heads*head_dim] rows (a view into qkv is fine); out [n, heads*head_dim]."""
    _rows(q, "attention q")
    n = q.shape[0]
    if out.shape != (n, heads * head_dim) or not out.is_contiguous() or out.dtype != q.dtype:
        raise KernelError("attention: out must be contiguous [n, heads*head_dim] of q's dtype")
    _check_pools("attention", q, tables, k_pool, v_pool, kv_heads, head_dim, page_size)
    check(
        load().shk_attention(
            _dev(q, "q"), q.stride(0), _dev(out, "out"), dtype_code(q.dtype), n, heads, kv_heads,
            head_dim, _dev(positions, "positions", torch.int32),
            _dev(token_seq, "token_seq", torch.int32), _dev(tables, "tables", torch.int32),
            tables.shape[1], tables.shape[0], _dev(k_pool, "k_pool"), _dev(v_pool, "v_pool"),
            page_size, k_pool.shape[0], int(window or 0), float(scale), _stream(),
        )
    )


def attention_supports_mfma(heads, kv_heads, head_dim, page_size, q_stride) -> bool:
    return bool(load().shk_attention_supports_mfma(heads, kv_heads, head_dim, page_size, q_stride))


def attention_decode(q, out, num_seqs, heads, kv_heads, head_dim, positions, tables, k_pool, v_pool,
                     page_size, window, scale, partial, nsplit, streaming=False) -> None:
    """bfloat16 MFMA attention for the first num_seqs rows of q, one token per sequence.
    `streaming`: fetch keys and values with non-temporal loads (same result; faster when
    the launch reads tens of megabytes of them)."""
    _rows(q, "attention_decode q")
    if q.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise KernelError("attention_decode: bfloat16 only")
    if q.shape[0] < num_seqs or tables.shape[0] < num_seqs or positions.shape[0] < num_seqs:
        raise KernelError("attention_decode: fewer rows than sequences")
    if out.shape[0] < num_seqs or out.shape[1] != heads * head_dim or not out.is_contiguous():
        raise KernelError("attention_decode: out must be contiguous [>= num_seqs, heads*head_dim]")
    _check_pools("attention_decode", q, tables, k_pool, v_pool, kv_heads, head_dim, page_size)
    if partial.numel() < num_seqs * heads * nsplit * (head_dim + 2):
        raise KernelError("attention_decode: partial scratch is too small")
    check(
        load().shk_attention_decode_bf16(
            _dev(q, "q"), q.stride(0), _dev(out, "out"), num_seqs, heads, kv_heads, head_dim,
            _dev(positions, "positions", torch.int32), _dev(tables, "tables", torch.int32),
            tables.shape[1], _dev(k_pool, "k_pool"), _dev(v_pool, "v_pool"), page_size,
            int(window or 0), float(scale), _dev(partial, "partial", torch.float32), nsplit,
            int(bool(streaming)), _stream(),
        )
    )


def attention_prefill(q, out, num_tiles, heads, kv_heads, head_dim, cu_q, ctx_lens, tile_seq, tile_q0,
                      tables, k_pool, v_pool, page_size, window, scale) -> None:
    """bfloat16 MFMA attention for prompt portions, in tiles of 16 queries."""
    _rows(q, "attention_prefill q")
    if q.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise KernelError("attention_prefill: bfloat16 only")
    if out.shape != (q.shape[0], heads * head_dim) or not out.is_contiguous():
        raise KernelError("attention_prefill: out must be contiguous [n, heads*head_dim]")
    if tile_seq.shape[0] < num_tiles or tile_q0.shape[0] < num_tiles:
        raise KernelError("attention_prefill: tile arrays are shorter than num_tiles")
    _check_pools("attention_prefill", q, tables, k_pool, v_pool, kv_heads, head_dim, page_size)
    check(
        load().shk_attention_prefill_bf16(
            _dev(q, "q"), q.stride(0), _dev(out, "out"), num_tiles, heads, kv_heads, head_dim,
            _dev(cu_q, "cu_q", torch.int32), _dev(ctx_lens, "ctx_lens", torch.int32),
            _dev(tile_seq, "tile_seq", torch.int32), _dev(tile_q0, "tile_q0", torch.int32),
            _dev(tables, "tables", torch.int32), tables.shape[1], _dev(k_pool, "k_pool"),
            _dev(v_pool, "v_pool"), page_size, int(window or 0), float(scale), _stream(),
        )
    )


def attention_prefill_shared_tiles(heads, kv_heads, head_dim, small=False) -> int:
    """16-query tiles per workgroup of attention_prefill_shared (`small`: of its
    variant with half as many wavefronts); 0 if the shape is not served."""
    return int(load().shk_attention_prefill_shared_tiles(heads, kv_heads, head_dim, int(small)))


def attention_prefill_shared(q, out, num_wgs, heads, kv_heads, head_dim, cu_q, ctx_lens, wg_seq, wg_q0,
                             tables, k_pool, v_pool, page_size, window, scale, small=False,
                             partial=None, nsplit: int = 1, first_token: int = 0) -> None:
    """bfloat16 MFMA attention for prompt portions; one workgroup per (run of query
    tiles, key/value head) shares each chunk of keys among its query heads.
    wg_seq / wg_q0 are in steps of 16 * attention_prefill_shared_tiles(..., small),
    launched in the list's order.  nsplit > 1 shares every entry's keys among
    that many workgroups, whose results pass through `partial` (float32, (rows
    of q from first_token on) * heads * nsplit * (head_dim + 2) values)."""
    _rows(q, "attention_prefill_shared q")
    if q.dtype != torch.bfloat16 or out.dtype != torch.bfloat16:
        raise KernelError("attention_prefill_shared: bfloat16 only")
    if out.shape != (q.shape[0], heads * head_dim) or not out.is_contiguous():
        raise KernelError("attention_prefill_shared: out must be contiguous [n, heads*head_dim]")
    if wg_seq.shape[0] < num_wgs or wg_q0.shape[0] < num_wgs:
        raise KernelError("attention_prefill_shared: workgroup arrays are shorter than num_wgs")
    _check_pools("attention_prefill_shared", q, tables, k_pool, v_pool, kv_heads, head_dim, page_size)
    prompt_tokens = q.shape[0] - first_token
    if nsplit > 1:
        need = prompt_tokens * heads * nsplit * (head_dim + 2)
        if partial is None or partial.dtype != torch.float32 or partial.numel() < need or prompt_tokens <= 0:
            raise KernelError(f"attention_prefill_shared: {nsplit} key splits need a float32 partial buffer "
                              f"of {need} values for the {prompt_tokens} prompt tokens")
    check(
        load().shk_attention_prefill_shared_bf16(
            _dev(q, "q"), q.stride(0), _dev(out, "out"), num_wgs, heads, kv_heads, head_dim,
            _dev(cu_q, "cu_q", torch.int32), _dev(ctx_lens, "ctx_lens", torch.int32),
            _dev(wg_seq, "wg_seq", torch.int32), _dev(wg_q0, "wg_q0", torch.int32),
            _dev(tables, "tables", torch.int32), tables.shape[1], _dev(k_pool, "k_pool"),
            _dev(v_pool, "v_pool"), page_size, int(window or 0), float(scale), int(small),
            _dev(partial, "partial", torch.float32) if nsplit > 1 else None, int(nsplit), int(first_token),
            int(prompt_tokens), _stream(),
        )
    )


_ARGMAX_SCRATCH: dict = {}


def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    """out[r] = lowest index of the maximum of logits[r]; logits float32 [rows, vocab]."""
    _rows(logits, "argmax logits")
    rows, vocab = logits.shape
    need = load().shk_argmax_scratch_floats(rows, vocab)
    scratch = None
    if need:
        key = (logits.device.type, logits.device.index)
        scratch = _ARGMAX_SCRATCH.get(key)
        if scratch is None or scratch.numel() < need:
            scratch = torch.empty(max(need, 1 << 16), dtype=torch.float32, device=logits.device)
            _ARGMAX_SCRATCH[key] = scratch
    check(load().shk_argmax(_dev(logits, "logits", torch.float32), _dev(out, "out", torch.int32),
                            rows, vocab, logits.stride(0),
                            None if scratch is None else scratch.data_ptr(), _stream()))


def sample_scratch_floats(rows: int, vocab: int) -> int:
    """float32 elements of scratch that sample() needs for logits [rows, vocab]."""
    return int(load().shk_sample_scratch_floats(rows, vocab))


def sample(logits, out, temperature, top_p, uniforms, scratch, nucleus: bool = True) -> None:
    """One token per row: argmax where temperature is 0, else a top-p draw with uniforms[r].
    nucleus=False promises that no row has a top_p below 1 (fewer passes)."""
    _rows(logits, "sample logits")
    rows, vocab = logits.shape
    if scratch.numel() < sample_scratch_floats(rows, vocab):
        raise KernelError(f"sample: scratch needs {sample_scratch_floats(rows, vocab)} float32 elements "
                          "(sample_scratch_floats)")
    check(
        load().shk_sample(
            _dev(logits, "logits", torch.float32), _dev(out, "out", torch.int32),
            _dev(temperature, "temperature", torch.float32), _dev(top_p, "top_p", torch.float32),
            _dev(uniforms, "uniforms", torch.float32), _dev(scratch, "scratch", torch.float32),
            scratch.numel(), rows, vocab, logits.stride(0), int(bool(nucleus)), _stream(),
        )
    )
