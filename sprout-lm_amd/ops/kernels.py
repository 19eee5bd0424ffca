"""One function per kernel entry point.  Host-side shape checks stand before every launch, because a
kernel that reads past a buffer can take the whole GPU down."""
from __future__ import annotations

import torch

from .library import KernelError, check, library

_CODES = {torch.float32: 0, torch.bfloat16: 1}


def _code(t: torch.Tensor, what: str) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"{what}: unsupported dtype {t.dtype}") from None


def _gpu(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise KernelError(f"{what} must live on the GPU; the engine has no CPU path.")
    if not t.is_contiguous():
        raise KernelError(f"{what} must be contiguous.")


def _ints(t: torch.Tensor, n: int, what: str) -> None:
    _gpu(t, what)
    if t.dtype != torch.int32 or t.numel() < n:
        raise KernelError(f"{what}: expected at least {n} int32 values, got {t.numel()} of {t.dtype}.")


_scope_stream: int | None = None    # the stream of the enclosing stream_scope, if any


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream if _scope_stream is None else _scope_stream


class stream_scope:
    """Looks the current HIP stream up once for every launch inside the `with` block.

    The lookup costs about as much as a launch itself, and a model step launches some two hundred
    kernels.  Entered anew inside a graph capture, it picks up the capturing stream.
    """

    def __enter__(self):
        global _scope_stream
        self._outer = _scope_stream
        _scope_stream = torch.cuda.current_stream().cuda_stream
        return self

    def __exit__(self, *exc):
        global _scope_stream
        _scope_stream = self._outer
        return False


def _ptr(t):
    return None if t is None else t.data_ptr()


# Variants of an operation that a part may ask for, as the C interface numbers them.  Only the listed ones have
# kernels; anything else is refused (KernelError) before a launch.
ROTARY_PAIRINGS = {"halves": 0}          # dimension d turns with d + rotary_dim / 2 ("neox")
GATE_ACTIVATIONS = {"silu": 0}
SCORE_STAGES = {"scaled_dot": 0}         # what stands between q . k and the softmax: the scale and nothing else
MAX_HEAD_DIM = 512                       # the largest head size any attention kernel takes


def variant_code(table: dict, name: str, what: str) -> int:
    try:
        return table[name]
    except KeyError:
        raise KernelError(f"No kernel for {what} {name!r}; there are kernels for: {sorted(table)}.") from None


def check_attention_sizes(heads: int, kv_heads: int, head_dim: int) -> None:
    """Raises KernelError unless some attention kernel takes these sizes (any page size goes with them).
    Head sizes of 16 ... 96 in steps of 16 and 128 run on the matrix cores in bfloat16, float32 in steps of 16 up
    to 256 on the matrix cores' float32 instructions, every other size up to 512 on the general kernel."""
    if kv_heads <= 0 or heads <= 0 or heads % kv_heads:
        raise KernelError(f"attention: {heads} query heads do not divide into {kv_heads} key/value heads")
    if not 0 < head_dim <= MAX_HEAD_DIM:
        raise KernelError(f"attention: head size {head_dim} is outside 1..{MAX_HEAD_DIM}, the sizes the kernels take")


def _check_pools(k_pool, v_pool, nkv: int, hd: int, dtype, what: str) -> tuple[int, int]:
    """Keys [pages, nkv, page_size, hd] and values [pages, nkv, hd, page_size]; returns (pages, page_size)."""
    _gpu(k_pool, "key pool"); _gpu(v_pool, "value pool")
    if k_pool.dim() != 4 or k_pool.shape[1] != nkv or k_pool.shape[3] != hd or k_pool.dtype != dtype:
        raise KernelError(f"{what}: key pool {tuple(k_pool.shape)} {k_pool.dtype} does not fit nkv={nkv} hd={hd} {dtype}")
    num_pages, _, page_size, _ = k_pool.shape
    if tuple(v_pool.shape) != (num_pages, nkv, hd, page_size) or v_pool.dtype != dtype:
        raise KernelError(f"{what}: value pool {tuple(v_pool.shape)} {v_pool.dtype} must be [{num_pages}, {nkv}, {hd}, {page_size}] {dtype}")
    return num_pages, page_size


def embed(table: torch.Tensor, tokens: torch.Tensor, residual: torch.Tensor) -> None:
    """residual[t] = table[tokens[t]] as float32."""
    _gpu(table, "embedding table"); _gpu(residual, "residual")
    T = residual.shape[0]
    V, H = table.shape
    _ints(tokens, T, "tokens")
    if residual.dtype != torch.float32 or residual.shape[1] != H:
        raise KernelError(f"embed: residual must be float32 [T, {H}], got {residual.dtype} {tuple(residual.shape)}")
    check(library().sp_embed(_stream(), _code(table, "embedding table"), table.data_ptr(), tokens.data_ptr(),
                             residual.data_ptr(), T, H, V))


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor, rows: torch.Tensor | None = None) -> None:
    """out[r] = rmsnorm(x[rows[r]] or x[r]) * weight; x is float32."""
    _gpu(x, "norm input"); _gpu(weight, "norm weight"); _gpu(out, "norm output")
    R, H = out.shape
    if x.dtype != torch.float32 or x.shape[1] != H or weight.numel() != H:
        raise KernelError(f"rmsnorm: shapes do not fit: x {tuple(x.shape)} {x.dtype}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    if rows is not None:
        _ints(rows, R, "norm rows")
    elif x.shape[0] < R:
        raise KernelError("rmsnorm: fewer input rows than output rows")
    check(library().sp_rmsnorm(_stream(), x.data_ptr(), _ptr(rows), _code(weight, "norm weight"), weight.data_ptr(),
                               float(eps), _code(out, "norm output"), out.data_ptr(), R, H))


STORE, ACCUMULATE, STORE_F32 = 0, 1, 2


def gemm(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor, bias: torch.Tensor | None = None,
         accumulate: bool = False) -> None:
    """out = a @ w.T (+ bias); with accumulate, out (float32) += a @ w.T (+ bias)."""
    _gpu(a, "gemm input"); _gpu(w, "gemm weight"); _gpu(out, "gemm output")
    T, K = a.shape
    N = w.shape[0]
    if w.shape[1] != K or tuple(out.shape) != (T, N):
        raise KernelError(f"gemm: shapes do not fit: a {tuple(a.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    if bias is not None:
        _gpu(bias, "gemm bias")
        if bias.numel() != N:
            raise KernelError(f"gemm: bias has {bias.numel()} values for {N} columns")
    if accumulate:
        if out.dtype != torch.float32:
            raise KernelError("gemm: accumulation needs a float32 output")
        mode = ACCUMULATE
    else:
        mode = STORE
    check(library().sp_gemm(_stream(), _code(a, "gemm input"), a.data_ptr(), _code(w, "gemm weight"), w.data_ptr(),
                            _code(bias, "gemm bias") if bias is not None else 0, _ptr(bias), mode,
                            _code(out, "gemm output"), out.data_ptr(), T, N, K))


def rope_cache(qkv: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor, rotary_dim: int, nq: int, nkv: int,
               hd: int, slot_mapping: torch.Tensor | None = None, k_pool: torch.Tensor | None = None,
               v_pool: torch.Tensor | None = None, inv_freq_tail: torch.Tensor | None = None, pairing: str = "halves") -> None:
    """Rotate q and k heads of qkv in place and write k, v into the pools (keys [pages, nkv, page, hd], values
    [pages, nkv, hd, page]).  `inv_freq_tail` (float32 qkv only): the float64 table minus `inv_freq`; with it
    angles, sines and cosines are computed in float64.  `pairing`: which dimensions turn together."""
    pairing_code = variant_code(ROTARY_PAIRINGS, pairing, "rotation pairing")
    _gpu(qkv, "qkv")
    T = qkv.shape[0]
    if qkv.shape[1] != (nq + 2 * nkv) * hd:
        raise KernelError(f"rope_cache: qkv has {qkv.shape[1]} columns, expected {(nq + 2 * nkv) * hd}")
    _ints(positions, T, "positions")
    _gpu(inv_freq, "inv_freq")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() < max(rotary_dim // 2, 0):
        raise KernelError("rope_cache: inv_freq must hold rotary_dim / 2 float32 values")
    if inv_freq_tail is not None:
        _gpu(inv_freq_tail, "inv_freq_tail")
        if inv_freq_tail.dtype != torch.float32 or inv_freq_tail.numel() != inv_freq.numel():
            raise KernelError("rope_cache: inv_freq_tail must be float32 and as long as inv_freq")
    page_size = num_pages = 0
    if nkv:
        _ints(slot_mapping, T, "slot_mapping")
        num_pages, page_size = _check_pools(k_pool, v_pool, nkv, hd, qkv.dtype, "rope_cache")
    check(library().sp_rope_cache(_stream(), _code(qkv, "qkv"), qkv.data_ptr(), positions.data_ptr(), inv_freq.data_ptr(),
                                  _ptr(inv_freq_tail), rotary_dim, _ptr(slot_mapping), _ptr(k_pool), _ptr(v_pool), T, nq, nkv, hd, page_size,
                                  num_pages, pairing_code))


TILE_SIZES = (16, 32, 64)   # query-tile sizes an attention kernel may ask for


def attention_lists(q_lens) -> dict:
    """Host-side work lists of a batch for the attention kernels (numpy int32 arrays).

    tiles_all_<n>: (sequence, first query) of every tile of n queries, over all sequences;
    tiles_multi_<n>: the same over the sequences with more than one query; decode_seqs: the others.
    """
    import numpy as np
    out = {}
    for n in TILE_SIZES:
        every = [(s, off) for s, q in enumerate(q_lens) for off in range(0, q, n)]
        out[f"tiles_all_{n}"] = np.asarray(every, dtype=np.int32).reshape(-1, 2)
        multi = [(s, off) for s, q in enumerate(q_lens) if q > 1 for off in range(0, q, n)]
        out[f"tiles_multi_{n}"] = np.asarray(multi, dtype=np.int32).reshape(-1, 2)
    out["decode_seqs"] = np.asarray([s for s, q in enumerate(q_lens) if q == 1], dtype=np.int32)
    return out


def mean_tile_walk(q_lens, ctx_lens, tile: int = 32) -> int:
    """Mean over the tiles of `tile` queries (of sequences with more than one query) of the keys a tile walks."""
    tiles = walked = 0
    for q, c in zip(q_lens, ctx_lens):
        q, c = int(q), int(c)
        if q > 1:
            n = -(-q // tile)
            tiles += n
            walked += n * (c - q) + tile * n * (n + 1) // 2     # the last tile counted as a whole one
    return walked // tiles if tiles else 0


class AttentionBatch:
    """The device-side description of a step's sequences that `attention` reads."""

    def __init__(self, q_start, q_len, ctx_len, n_seqs: int, lists: dict, max_decode_ctx: int, max_ctx: int,
                 mean_walk: int = 0):
        """`lists`: name -> (device int32 tensor, number of entries), names as in `attention_lists`;
        `max_decode_ctx`, `max_ctx`: the longest context among one-query sequences, and among all;
        `mean_walk`: the mean number of keys that a tile of queries walks, see `mean_tile_walk` (a hint for
        how the kernels share out the work; unknown: 0)."""
        self.q_start, self.q_len, self.ctx_len, self.n_seqs = q_start, q_len, ctx_len, n_seqs
        self.lists, self.max_decode_ctx, self.max_ctx = lists, max_decode_ctx, max_ctx
        self.mean_walk = mean_walk

    @classmethod
    def build(cls, q_lens, ctx_lens, device) -> "AttentionBatch":
        """From host lists, one upload per array (tests and small tools; the engine packs its own)."""
        import numpy as np
        to = lambda a: torch.as_tensor(np.ascontiguousarray(a), dtype=torch.int32).to(device)
        starts = np.concatenate([[0], np.cumsum(q_lens)[:-1]]) if len(q_lens) else np.zeros(0)
        lists = {k: (to(v), len(v)) for k, v in attention_lists(q_lens).items()}
        decode_ctx = [c for c, q in zip(ctx_lens, q_lens) if q == 1]
        return cls(to(starts), to(q_lens), to(ctx_lens), len(q_lens), lists, max(decode_ctx, default=0),
                   max((int(c) for c in ctx_lens), default=0),
                   mean_tile_walk(q_lens, ctx_lens))


def attention_plan(dtype: torch.dtype, hd: int, page_size: int, nq: int, nkv: int, kind: int = 0) -> tuple[int, bool]:
    """(queries per tile, whether the tile list must hold every sequence) of the kernel that will run."""
    import ctypes
    plan = (ctypes.c_int * 2)()
    check(library().sp_attention_plan(_CODES[dtype], hd, page_size, nq, nkv, kind, plan))
    return plan[0], bool(plan[1])


def attention(q: torch.Tensor, q_stride: int, k_pool: torch.Tensor, v_pool: torch.Tensor, block_tables: torch.Tensor,
              batch: AttentionBatch, out: torch.Tensor, nq: int, nkv: int, hd: int, window: int | None, scale: float,
              workspace=None, kind: int = 0, project=None, scores: str = "scaled_dot") -> bool:
    """Causal attention of a mixed batch over paged keys and values (see sprout_hip.h).

    `workspace(n)` must return a float32 device tensor of at least n elements (default: a new one).
    `project`: (w_o [hidden, nq * hd], residual float32 [T, hidden]) of an output projection without bias
    that may be folded in: where the kernels take the step that way (one-query sequences only, bfloat16),
    residual += attention . w_o^T, `out` is left untouched and True is returned; otherwise False, and the
    projection is the caller's.
    """
    scores_code = variant_code(SCORE_STAGES, scores, "score stage")
    for t, what in ((q, "q"), (out, "attention output")):
        _gpu(t, what)
    T = out.shape[0]
    if out.shape[1] != nq * hd or q.shape[0] < T or q.dtype != out.dtype:
        raise KernelError(f"attention: shapes or dtypes do not fit: q {tuple(q.shape)} {q.dtype}, out {tuple(out.shape)} {out.dtype}")
    if q_stride > q.shape[1] or q_stride < nq * hd:
        raise KernelError("attention: bad q row stride")
    if nkv <= 0 or nq % nkv:
        raise KernelError(f"attention: {nq} query heads do not divide into {nkv} groups")
    check_attention_sizes(nq, nkv, hd)
    num_pages, page_size = _check_pools(k_pool, v_pool, nkv, hd, q.dtype, "attention")
    _gpu(block_tables, "block tables")
    n_seqs = batch.n_seqs
    if block_tables.dtype != torch.int32 or block_tables.dim() != 2 or block_tables.shape[0] < n_seqs:
        raise KernelError("attention: block tables must be int32 [sequences, max_blocks]")
    for t, what in ((batch.q_start, "q_start"), (batch.q_len, "q_len"), (batch.ctx_len, "ctx_len")):
        _ints(t, n_seqs, what)
    tile_q, every = attention_plan(q.dtype, hd, page_size, nq, nkv, kind)
    tiles, n_tiles = batch.lists[f"tiles_{'all' if every else 'multi'}_{tile_q}"]
    decode, n_decode = (None, 0) if every else batch.lists["decode_seqs"]
    _ints(tiles, 2 * n_tiles, "tiles")
    max_decode_ctx = batch.max_decode_ctx if n_decode else 0
    # a kernel that takes every sequence in its tile list is told when each of them brings one query
    one_query_each = every and n_tiles == n_seqs and batch.lists[f"tiles_multi_{tile_q}"][1] == 0
    if n_decode:
        if decode is not None:         # None: sequences 0 .. n_decode - 1
            _ints(decode, n_decode, "decode_seqs")
        elif n_decode != n_seqs or n_tiles:
            # the kernels then take sequence i's query to be row i
            raise KernelError("attention: without a decode list every sequence must bring one query")
        if max_decode_ctx > block_tables.shape[1] * page_size:
            raise KernelError("attention: a decode context is longer than its block table")
    if n_tiles and batch.max_ctx > block_tables.shape[1] * page_size:
        raise KernelError(f"attention: a context of {batch.max_ctx} tokens is longer than its block table "
                          f"({block_tables.shape[1]} pages of {page_size})")
    max_tile_ctx = batch.max_ctx if n_tiles else 0
    if one_query_each:
        n_decode = n_tiles
    need = library().sp_attention_workspace_floats(_code(q, "q"), hd, page_size, nq, nkv, kind, n_decode, max_decode_ctx,
                                                   n_tiles, max_tile_ctx)
    ws = None
    if need:
        ws = workspace(need) if workspace is not None else torch.empty(need, dtype=torch.float32, device=q.device)
        if ws.dtype != torch.float32 or ws.numel() < need:
            raise KernelError("attention: workspace too small")
    if project is not None and kind == 0 and n_tiles == 0 and n_decode and need and q.dtype == torch.bfloat16 and not every:
        w_o, residual = project
        hidden = w_o.shape[0]
        if (w_o.dtype == torch.bfloat16 and w_o.is_contiguous() and tuple(w_o.shape) == (hidden, nq * hd)
                and residual.dtype == torch.float32 and residual.is_contiguous() and residual.dim() == 2
                and residual.shape[1] == hidden and residual.shape[0] >= T
                and library().sp_attention_decode_project_takes(hd, page_size, nq, nkv, n_decode, max_decode_ctx, hidden)):
            _gpu(w_o, "w_o"); _gpu(residual, "residual")
            check(library().sp_attention_decode_project(
                _stream(), q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(), block_tables.data_ptr(),
                block_tables.shape[1], batch.q_start.data_ptr(), batch.ctx_len.data_ptr(),
                _ptr(decode) if decode is not None else None, n_decode, max_decode_ctx, _ptr(ws), need, w_o.data_ptr(),
                residual.data_ptr(), hidden, nq, nkv, hd, page_size, num_pages, int(window) if window else 0,
                float(scale), scores_code))
            return True
    check(library().sp_attention(_stream(), _code(q, "q"), q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
                                 block_tables.data_ptr(), block_tables.shape[1], batch.q_start.data_ptr(),
                                 batch.q_len.data_ptr(), batch.ctx_len.data_ptr(), _ptr(tiles) if n_tiles else None,
                                 n_tiles, tile_q, max_tile_ctx, int(batch.mean_walk),
                                 _ptr(decode) if n_decode and decode is not None else None, n_decode,
                                 max_decode_ctx, _ptr(ws),
                                 need, out.data_ptr(), nq, nkv, hd, page_size, num_pages, int(window) if window else 0,
                                 float(scale), kind, scores_code))
    return False


def feed_tokens(tokens: torch.Tensor, previous: torch.Tensor, source: torch.Tensor, vocab: int) -> None:
    """tokens[i] = previous[source[i]] where source[i] >= 0: tokens of a step the host has not read yet."""
    n = tokens.numel()
    _ints(tokens, n, "tokens"); _ints(source, n, "token sources"); _ints(previous, 1, "sampled tokens")
    check(library().sp_feed_tokens(_stream(), tokens.data_ptr(), previous.data_ptr(), source.data_ptr(), n, int(vocab)))


FUSED_ROPE, FUSED_SILU = 3, 4


def fused_supported(kind: int, T: int, N: int, K: int, hd: int = 0, rotary_dim: int = 0, norm: bool = False,
                    variant: str | None = None) -> bool:
    """Whether the fused kernels take this shape (see sprout_hip.h).  `variant`: the rotation's pairing
    (FUSED_ROPE) or the gate's activation (FUSED_SILU) by name; one without a kernel is not taken."""
    code = 0
    if variant is not None:
        code = (ROTARY_PAIRINGS if kind == FUSED_ROPE else GATE_ACTIVATIONS).get(variant, -1)
    return bool(library().sp_fused_supported(kind, T, N, K, hd, rotary_dim, int(norm), code))


def fused_norm_pays(T: int, N: int, K: int) -> bool:
    """Whether the norm folded into the product beats a norm kernel of its own followed by the product."""
    return bool(library().sp_fused_norm_pays(T, N, K))


PLAN_STORE, PLAN_ACCUMULATE, PLAN_GATED, PLAN_ROTATING = 0, 1, 2, 3


def pipe_plan(kind: int, T: int, N: int, K: int, hd: int = 0):
    """(block rows, block columns, splits of K, waves of a block) that the tiled product for many tokens would take
    for T x N x K, or None where that kernel (for PLAN_ROTATING its rotating epilogue) does not take the product.
    Runs nothing and needs no GPU."""
    import ctypes
    plan = (ctypes.c_int * 4)()
    if library().sp_pipe_plan(kind, T, N, K, hd, plan):
        return None
    return tuple(plan)


def pipe_tiles(tiles_t: int, tiles_n: int) -> list:
    """For every block of the tiled product's launch over tiles_t token tiles and tiles_n weight tiles, in the order
    of the blocks (block b runs on XCD b % 8): (token tile, weight tile), or None for a block with nothing to do.
    Runs nothing and needs no GPU."""
    import ctypes
    blocks = library().sp_pipe_tiles(tiles_t, tiles_n, (ctypes.c_int * 2)(), 0)
    if blocks < 0:
        raise KernelError(f"sp_pipe_tiles: no tiles for {tiles_t} x {tiles_n}")
    out = (ctypes.c_int * (2 * blocks))()
    library().sp_pipe_tiles(tiles_t, tiles_n, out, blocks)
    return [None if out[2 * b] < 0 else (out[2 * b], out[2 * b + 1]) for b in range(blocks)]


def _activations(x, residual, norm_weight, K: int, what: str):
    """Checks the two ways activations reach a fused kernel; returns (x ptr, residual ptr, norm dtype, norm ptr, T)."""
    if residual is not None:
        _gpu(residual, "residual"); _gpu(norm_weight, "norm weight")
        if residual.dtype != torch.float32 or residual.shape[1] != K or norm_weight.numel() != K:
            raise KernelError(f"{what}: residual must be float32 [T, {K}] with a norm weight of {K}")
        return None, residual.data_ptr(), _code(norm_weight, "norm weight"), norm_weight.data_ptr(), residual.shape[0]
    _gpu(x, "activations")
    if x.dtype != torch.bfloat16 or x.shape[1] != K:
        raise KernelError(f"{what}: activations must be bfloat16 [T, {K}], got {x.dtype} {tuple(x.shape)}")
    return x.data_ptr(), None, 0, None, x.shape[0]


def qkv_rope_cache(w: torch.Tensor, bias, q_out: torch.Tensor, positions, inv_freq, rotary_dim: int, slot_mapping,
                   k_pool, v_pool, nq: int, nkv: int, hd: int, x=None, residual=None, norm_weight=None,
                   eps: float = 0.0, table=None, pairing: str = "halves") -> None:
    """q, k, v = activations . w^T + bias; rotate q and k; q to q_out, k and v into the paged pools.

    Activations are x (bfloat16) or rmsnorm(residual) * norm_weight computed inside the kernel.
    `table`: `rope_table` of these positions (float32 [T, hd / 2, 2]), which the many-token kernel reads
    instead of computing sines and cosines."""
    _gpu(w, "qkv weight"); _gpu(q_out, "q output")
    N, K = w.shape
    xp, rp, nd, npt, T = _activations(x, residual, norm_weight, K, "qkv_rope_cache")
    if w.dtype != torch.bfloat16 or N != (nq + 2 * nkv) * hd or tuple(q_out.shape) != (T, nq * hd) or q_out.dtype != torch.bfloat16:
        raise KernelError("qkv_rope_cache: weight or q output does not fit the head counts")
    if bias is not None:
        _gpu(bias, "qkv bias")
        if bias.numel() != N:
            raise KernelError("qkv_rope_cache: bias size")
    _ints(positions, T, "positions"); _ints(slot_mapping, T, "slot_mapping"); _gpu(inv_freq, "inv_freq")
    _, page_size = _check_pools(k_pool, v_pool, nkv, hd, torch.bfloat16, "qkv_rope_cache")
    if table is not None:
        _gpu(table, "rotation table")
        if table.dtype != torch.float32 or tuple(table.shape) != (T, hd // 2, 2) or rotary_dim != hd:
            raise KernelError(f"qkv_rope_cache: the rotation table must be float32 [{T}, {hd // 2}, 2]")
    check(library().sp_qkv_rope_cache(_stream(), xp, rp, nd, npt, float(eps), w.data_ptr(),
                                      _code(bias, "bias") if bias is not None else 0, _ptr(bias), q_out.data_ptr(),
                                      positions.data_ptr(), inv_freq.data_ptr(), rotary_dim, slot_mapping.data_ptr(),
                                      k_pool.data_ptr(), v_pool.data_ptr(), T, K, nq, nkv, hd, page_size, _ptr(table),
                                      variant_code(ROTARY_PAIRINGS, pairing, "rotation pairing")))


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, out: torch.Tensor) -> None:
    """out[t, d] = (cos, sin) of positions[t] * inv_freq[d]; out float32 [T, len(inv_freq), 2]."""
    _gpu(inv_freq, "inv_freq"); _gpu(out, "rotation table")
    T, half = out.shape[0], inv_freq.numel()
    _ints(positions, T, "positions")
    if inv_freq.dtype != torch.float32 or out.dtype != torch.float32 or tuple(out.shape) != (T, half, 2):
        raise KernelError("rope_table: inv_freq float32 [half] and out float32 [T, half, 2] expected")
    check(library().sp_rope_table(_stream(), positions.data_ptr(), inv_freq.data_ptr(), half, out.data_ptr(), T))


def gate_up_silu(w: torch.Tensor, out: torch.Tensor, x=None, residual=None, norm_weight=None, eps: float = 0.0,
                 activation: str = "silu") -> None:
    """out = act(a . w[:I]^T) * (a . w[I:]^T) for activations a as in `qkv_rope_cache`."""
    _gpu(w, "gate/up weight"); _gpu(out, "gated output")
    N, K = w.shape
    xp, rp, nd, npt, T = _activations(x, residual, norm_weight, K, "gate_up_silu")
    if w.dtype != torch.bfloat16 or N % 2 or tuple(out.shape) != (T, N // 2) or out.dtype != torch.bfloat16:
        raise KernelError("gate_up_silu: weight [2 I, K] and output [T, I] bfloat16 expected")
    check(library().sp_gate_up_silu(_stream(), xp, rp, nd, npt, float(eps), w.data_ptr(), out.data_ptr(), T, N // 2, K,
                                    variant_code(GATE_ACTIVATIONS, activation, "gate activation")))


def gate_up_silu_f32(w: torch.Tensor, x: torch.Tensor, out: torch.Tensor, activation: str = "silu", norm_weight=None,
                     eps: float = 0.0) -> bool:
    """out = act(a . w[:I]^T) * (a . w[I:]^T), everything float32, for the few tokens of a decode step; a = x, or
    rmsnorm(x) * norm_weight computed inside the kernel where norm_weight is given (x is then the residual).  Returns
    False (and does nothing) where the kernel does not take the shape: the caller then multiplies and gates in turn."""
    N, K = w.shape
    T, I = out.shape
    if (w.dtype != torch.float32 or x.dtype != torch.float32 or out.dtype != torch.float32 or N != 2 * I
            or tuple(x.shape) != (T, K) or not library().sp_gate_up_silu_f32_takes(T, I, K)):
        return False
    if norm_weight is not None and (norm_weight.dtype != torch.float32 or norm_weight.numel() != K):
        return False
    _gpu(w, "gate/up weight"); _gpu(x, "activations"); _gpu(out, "gated output")
    check(library().sp_gate_up_silu_f32(_stream(), x.data_ptr(), _ptr(norm_weight), float(eps), w.data_ptr(), out.data_ptr(),
                                        T, I, K, variant_code(GATE_ACTIVATIONS, activation, "gate activation")))
    return True


def qkv_rope_cache_f32(w: torch.Tensor, bias, x: torch.Tensor, q_out: torch.Tensor, positions, inv_freq, inv_freq_tail,
                       rotary_dim: int, slot_mapping, k_pool, v_pool, nq: int, nkv: int, hd: int, norm_weight=None,
                       eps: float = 0.0, pairing: str = "halves") -> bool:
    """The float32 path's q/k/v product of a decode step with bias, rotation and cache write folded in (and the norm
    before it, where norm_weight is given and x is the residual); see sprout_hip.h.  Returns False, and does
    nothing, where the kernel does not take the shape."""
    N, K = w.shape
    T = x.shape[0]
    code = ROTARY_PAIRINGS.get(pairing, -1)
    if (w.dtype != torch.float32 or x.dtype != torch.float32 or q_out.dtype != torch.float32 or N != (nq + 2 * nkv) * hd
            or tuple(x.shape) != (T, K) or tuple(q_out.shape) != (T, nq * hd) or k_pool is None or k_pool.dtype != torch.float32
            or not library().sp_qkv_rope_cache_f32_takes(T, K, nq, nkv, hd, rotary_dim, code)):
        return False
    if norm_weight is not None and (norm_weight.dtype != torch.float32 or norm_weight.numel() != K):
        return False
    for t_, what in ((w, "qkv weight"), (x, "activations"), (q_out, "q output"), (inv_freq, "inv_freq")):
        _gpu(t_, what)
    if bias is not None:
        _gpu(bias, "qkv bias")
        if bias.numel() != N:
            raise KernelError("qkv_rope_cache_f32: bias size")
    if inv_freq.dtype != torch.float32 or inv_freq.numel() < hd // 2 or (inv_freq_tail is not None and (
            inv_freq_tail.dtype != torch.float32 or inv_freq_tail.numel() != inv_freq.numel())):
        raise KernelError("qkv_rope_cache_f32: inv_freq (and its tail) must hold hd / 2 float32 values")
    _ints(positions, T, "positions"); _ints(slot_mapping, T, "slot_mapping")
    num_pages, page_size = _check_pools(k_pool, v_pool, nkv, hd, torch.float32, "qkv_rope_cache_f32")
    check(library().sp_qkv_rope_cache_f32(_stream(), x.data_ptr(), _ptr(norm_weight), float(eps), w.data_ptr(),
                                          _code(bias, "bias") if bias is not None else 0, _ptr(bias), q_out.data_ptr(),
                                          positions.data_ptr(), inv_freq.data_ptr(), _ptr(inv_freq_tail), rotary_dim,
                                          slot_mapping.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(), T, K, nq, nkv, hd,
                                          page_size, num_pages, code))
    return True


def silu_mul(gu: torch.Tensor, out: torch.Tensor, activation: str = "silu") -> None:
    """out[t, i] = act(gu[t, i]) * gu[t, I + i]."""
    _gpu(gu, "gate/up"); _gpu(out, "gated output")
    T, I = out.shape
    if tuple(gu.shape) != (T, 2 * I) or gu.dtype != out.dtype:
        raise KernelError(f"silu_mul: shapes do not fit: gu {tuple(gu.shape)}, out {tuple(out.shape)}")
    check(library().sp_silu_mul(_stream(), _code(gu, "gate/up"), gu.data_ptr(), out.data_ptr(), T, I,
                                variant_code(GATE_ACTIVATIONS, activation, "gate activation")))


def random_fill(dst: torch.Tensor, key: int, scale: float, offset: float | None = None, first: int = 0) -> None:
    """dst (flat order) = the seeded values of elements first .. of the tensor keyed `key` (see sprout_hip.h)."""
    _gpu(dst, "random fill destination")
    check(library().sp_random_fill(_stream(), _code(dst, "random fill destination"), dst.data_ptr(), dst.numel(),
                                   key & 0xFFFFFFFFFFFFFFFF, first, float(scale), float(offset or 0.0), int(offset is not None)))


def sample_workspace_floats(rows: int, vocab: int) -> int:
    return library().sp_sample_workspace_floats(rows, vocab)


def sample(logits: torch.Tensor, out: torch.Tensor, workspace: torch.Tensor, temperature: torch.Tensor | None = None,
           seed: torch.Tensor | None = None, counter: torch.Tensor | None = None) -> None:
    """out[r] = sampled token of row r (greedy where temperature is 0 or absent), -1 for a non-finite row."""
    _gpu(logits, "logits"); _gpu(out, "sampled tokens"); _gpu(workspace, "sampling workspace")
    R, V = logits.shape
    if logits.dtype != torch.float32 or out.dtype != torch.int32 or out.numel() < R:
        raise KernelError("sample: logits must be float32 and the output int32 with one entry per row")
    if workspace.dtype != torch.float32 or workspace.numel() < sample_workspace_floats(R, V):
        raise KernelError("sample: workspace too small")
    if temperature is not None:
        _gpu(temperature, "temperature"); _gpu(seed, "seed"); _ints(counter, R, "counter")
        if temperature.dtype != torch.float32 or temperature.numel() < R or seed.dtype != torch.int64 or seed.numel() < R:
            raise KernelError("sample: temperature must be float32 and seed int64, one per row")
    check(library().sp_sample(_stream(), logits.data_ptr(), _ptr(temperature), _ptr(seed), _ptr(counter), out.data_ptr(),
                              workspace.data_ptr(), R, V))


def probe_machine(device=None, megabytes: int = 4096, repeats: int = 5) -> dict:
    """What this GPU gives a kernel that only reads memory (GB/s) and one that only multiplies bfloat16 on the
    matrix cores (TFLOP/s): the best of a few runs of the library's two probe kernels, for reports that set a
    measured rate beside the published peak."""
    import ctypes
    lib = library()
    device = device or torch.device("cuda", torch.cuda.current_device())
    data = torch.zeros(megabytes << 20, dtype=torch.uint8, device=device)
    sink = torch.zeros(4, dtype=torch.float32, device=device)
    flops = ctypes.c_double()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best_read = best_mfma = float("inf")
    for _ in range(repeats + 1):       # the first run warms up
        for blocks in (1024, 2048, 4096, 8192):     # how many blocks read fastest differs a little from box to box
            start.record()
            check(lib.sp_probe_read(_stream(), data.data_ptr(), data.numel(), blocks, sink.data_ptr()))
            stop.record(); stop.synchronize()
            best_read = min(best_read, start.elapsed_time(stop))
        start.record()
        check(lib.sp_probe_mfma(_stream(), 256 * 8, 20000, sink.data_ptr(), ctypes.byref(flops)))
        stop.record(); stop.synchronize()
        best_mfma = min(best_mfma, start.elapsed_time(stop))
    return {"hbm_read_gbs": round(data.numel() / best_read / 1e6, 1), "mfma_bf16_tflops": round(flops.value / best_mfma / 1e9, 1)}
