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
ROTARY_PAIRINGS = {"halves": 0}          # dimension d turns with d + rotary_dim / 2 ("neox"); the latent mixer's own
                                         # kernel (latent_prepare) turns neighbours (2i, 2i + 1)
GATE_ACTIVATIONS = {"silu": 0,           # silu(g) * u
                    "clamped_swish": 1,  # g' = min(g, limit), u' = clamp(u, -limit, limit): g' * sigmoid(1.702 g') * (u' + 1)
                    "relu": 2}           # max(g, 0) * u
SCORE_STAGES = {"scaled_dot": 0,         # what stands between q . k and the softmax: the scale and nothing else,
                "capped": 1}             # or the scaled product s squashed to cap * tanh(s / cap)
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


def layernorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor, rows: torch.Tensor | None = None,
              weight2: torch.Tensor | None = None, out2: torch.Tensor | None = None, bias: torch.Tensor | None = None,
              bias2: torch.Tensor | None = None) -> None:
    """out[r] = (x - mean) / sqrt(mean((x - mean)^2) + eps) * weight (+ bias) of x[rows[r]] or x[r]; x is float32.  With
    weight2 and out2 the same normalised row times a second weight (+ bias2) goes to out2 (two norms of one input in one
    pass)."""
    _gpu(x, "norm input"); _gpu(weight, "norm weight"); _gpu(out, "norm output")
    R, H = out.shape
    if x.dtype != torch.float32 or x.shape[1] != H or weight.numel() != H:
        raise KernelError(f"layernorm: shapes do not fit: x {tuple(x.shape)} {x.dtype}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    if (weight2 is None) != (out2 is None):
        raise KernelError("layernorm: a second weight goes with a second output")
    if weight2 is not None:
        _gpu(weight2, "second norm weight"); _gpu(out2, "second norm output")
        if weight2.dtype != weight.dtype or weight2.numel() != H or out2.dtype != out.dtype or tuple(out2.shape) != (R, H):
            raise KernelError("layernorm: the second weight and output must be shaped and typed like the first")
    for b, what in ((bias, "norm bias"), (bias2, "second norm bias")):
        if b is not None:
            _gpu(b, what)
            if b.dtype != weight.dtype or b.numel() != H:
                raise KernelError(f"layernorm: the {what} must be shaped and typed like the weight")
    if bias2 is not None and weight2 is None:
        raise KernelError("layernorm: a second bias goes with a second weight")
    if rows is not None:
        _ints(rows, R, "norm rows")
    elif x.shape[0] < R:
        raise KernelError("layernorm: fewer input rows than output rows")
    check(library().sp_layernorm(_stream(), x.data_ptr(), _ptr(rows), _code(weight, "norm weight"), weight.data_ptr(),
                                 _ptr(weight2), _ptr(bias), _ptr(bias2), float(eps), _code(out, "norm output"),
                                 out.data_ptr(), _ptr(out2), R, H))


def embed_bigram(table: torch.Tensor, pairs: torch.Tensor, tokens, positions, q_start, q_len, seq_of_token, state_slots,
                 last_token: torch.Tensor, residual: torch.Tensor, n_seqs: int, buckets: int, mul_prev: int, mul_cur: int) -> None:
    """residual[t] = table[tokens[t]] + pairs[(previous * mul_prev + tokens[t] * mul_cur) % buckets] (row `buckets` at
    position 0) as float32.  `last_token` (int32, one entry per state slot) carries a sequence's last token from step
    to step."""
    _gpu(table, "embedding table"); _gpu(pairs, "pair table"); _gpu(residual, "residual"); _gpu(last_token, "last tokens")
    T = residual.shape[0]
    V, H = table.shape
    if residual.dtype != torch.float32 or residual.shape[1] != H:
        raise KernelError(f"embed_bigram: residual must be float32 [T, {H}], got {residual.dtype} {tuple(residual.shape)}")
    if tuple(pairs.shape) != (buckets + 1, H) or pairs.dtype != table.dtype:
        raise KernelError(f"embed_bigram: the pair table must be [{buckets + 1}, {H}] {table.dtype}, got {tuple(pairs.shape)} {pairs.dtype}")
    if last_token.dtype != torch.int32:
        raise KernelError("embed_bigram: last tokens must be int32")
    for t, n, what in ((tokens, T, "tokens"), (positions, T, "positions"), (seq_of_token, T, "seq_of_token"),
                       (q_start, n_seqs, "q_start"), (q_len, n_seqs, "q_len"), (state_slots, n_seqs, "state_slots")):
        _ints(t, n, what)
    check(library().sp_embed_bigram(_stream(), _code(table, "embedding table"), table.data_ptr(), pairs.data_ptr(),
                                    tokens.data_ptr(), positions.data_ptr(), q_start.data_ptr(), q_len.data_ptr(),
                                    seq_of_token.data_ptr(), state_slots.data_ptr(), last_token.data_ptr(),
                                    residual.data_ptr(), T, H, V, int(buckets), int(mul_prev), int(mul_cur)))


def latent_prepare(proj: torch.Tensor, q_off: int, heads: int, dim: int, rot: int, dkv_off: int, rank: int,
                   norm_weight: torch.Tensor, eps: float, positions, freq: torch.Tensor, rot_dims: int, magnitude: float,
                   slot_mapping, k_pool, v_pool, q_out: torch.Tensor) -> None:
    """From a row of projections: the normed latent and the turned shared key part into the pools (keys
    [pages, 1, page, rank + rot], values [pages, 1, rank + rot, page], whose last rot columns are left alone), and
    every head's turned query part into q_out[t, head, rank:] (see sprout_hip.h).  Float32 rows turn by float64 angles."""
    _gpu(proj, "projections"); _gpu(norm_weight, "latent norm weight"); _gpu(q_out, "latent queries"); _gpu(freq, "frequencies")
    T, stride = proj.shape
    width = rank + rot
    if tuple(q_out.shape) != (T, heads * width) or q_out.dtype != proj.dtype:
        raise KernelError(f"latent_prepare: queries must be [{T}, {heads * width}] {proj.dtype}, got {tuple(q_out.shape)} {q_out.dtype}")
    if norm_weight.numel() != rank or freq.dtype != torch.float64 or freq.numel() < rot_dims // 2:
        raise KernelError("latent_prepare: the norm weight must hold rank numbers and freq rot_dims / 2 float64 numbers")
    _ints(positions, T, "positions")
    page_size = num_pages = 0
    if slot_mapping is not None:
        _ints(slot_mapping, T, "slot_mapping")
        num_pages, page_size = _check_pools(k_pool, v_pool, 1, width, proj.dtype, "latent_prepare")
    check(library().sp_latent_prepare(_stream(), _code(proj, "projections"), proj.data_ptr(), stride, q_off, heads, dim, rot,
                                      dkv_off, rank, _code(norm_weight, "latent norm weight"), norm_weight.data_ptr(),
                                      float(eps), positions.data_ptr(), freq.data_ptr(), rot_dims, float(magnitude),
                                      int(proj.dtype == torch.float32), _ptr(slot_mapping), _ptr(k_pool), _ptr(v_pool),
                                      page_size, num_pages, q_out.data_ptr(), T))


def head_gemm(a: torch.Tensor, a_offset: int, a_head_stride: int, w: torch.Tensor, out: torch.Tensor, out_offset: int,
              out_head_stride: int, gate: torch.Tensor | None = None, gate_offset: int = 0) -> None:
    """Per head h: out[t, out_offset + h * out_head_stride + n] = sum_k a[t, a_offset + h * a_head_stride + k] * w[h, n, k],
    times sigmoid(gate[t, gate_offset + h]) where `gate` is given.  w [heads, N, K]; a, w, out (and gate) of one dtype."""
    _gpu(a, "head product input"); _gpu(w, "head product weight"); _gpu(out, "head product output")
    heads, N, K = w.shape
    T = out.shape[0]
    if a.dtype != w.dtype or out.dtype != w.dtype or a.shape[0] < T:
        raise KernelError(f"head_gemm: dtypes or rows do not fit: a {a.dtype} {tuple(a.shape)}, w {w.dtype}, out {out.dtype} {tuple(out.shape)}")
    if (a_offset < 0 or a_offset + (heads - 1) * a_head_stride + K > a.shape[1]
            or out_offset < 0 or out_offset + (heads - 1) * out_head_stride + N > out.shape[1]):
        raise KernelError(f"head_gemm: {heads} heads of K={K}, N={N} do not fit rows of {a.shape[1]} and {out.shape[1]}")
    size = a.element_size()
    gate_ptr, gate_stride = None, 0
    if gate is not None:
        _gpu(gate, "head gate")
        if gate.dtype != w.dtype or gate.shape[0] < T or gate_offset < 0 or gate_offset + heads > gate.shape[1]:
            raise KernelError("head_gemm: the gate does not hold a number per token and head")
        gate_ptr, gate_stride = gate.data_ptr() + gate_offset * size, gate.shape[1]
    check(library().sp_head_gemm(_stream(), _code(w, "head product weight"), a.data_ptr() + a_offset * size, a.shape[1],
                                 a_head_stride, w.data_ptr(), out.data_ptr() + out_offset * size, out.shape[1],
                                 out_head_stride, gate_ptr, gate_stride, T, heads, N, K))


def group_tile_rows(dtype: torch.dtype = torch.float32, rows: int = 0, groups: int = 1, eights: bool = False) -> int:
    """Rows a tile of the grouped products holds: 128 where the groups own at least that many rows each on average and
    the matrix-core kernels take the operands (bfloat16, every K in `eights`), else 64."""
    return library().sp_group_tile_rows(_CODES[dtype], int(rows), int(groups), 8 if eights else 1)


def route_max_tiles(pairs: int, experts: int, tile_rows: int = 64) -> int:
    return library().sp_route_max_tiles(pairs, experts, tile_rows)


def route_topk(logits: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor) -> None:
    """ids, weights [T, top] = the top largest logits of every row (falling; the lowest index wins a tie) and the
    softmax over those alone."""
    _gpu(logits, "router logits"); _gpu(ids, "chosen experts"); _gpu(weights, "expert weights")
    T, E = logits.shape
    top = ids.shape[1]
    if logits.dtype != torch.float32 or ids.dtype != torch.int32 or weights.dtype != torch.float32 or \
            tuple(ids.shape) != (T, top) or tuple(weights.shape) != (T, top) or not 0 < top <= E:
        raise KernelError("route_topk: float32 logits [T, E], int32 ids and float32 weights [T, top] expected")
    check(library().sp_route_topk(_stream(), logits.data_ptr(), ids.data_ptr(), weights.data_ptr(), T, E, top))


def route(logits: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, row_of_pair, pair_of_row, tiles, n_tiles,
          tile_rows: int = 64) -> None:
    """route_topk and route_sort in one call (one launch for steps of up to 256 tokens)."""
    _gpu(logits, "router logits"); _gpu(ids, "chosen experts"); _gpu(weights, "expert weights")
    T, E = logits.shape
    top = ids.shape[1]
    if logits.dtype != torch.float32 or ids.dtype != torch.int32 or weights.dtype != torch.float32 or \
            tuple(ids.shape) != (T, top) or tuple(weights.shape) != (T, top) or not 0 < top <= E:
        raise KernelError("route: float32 logits [T, E], int32 ids and float32 weights [T, top] expected")
    pairs = T * top
    _ints(row_of_pair, pairs, "row_of_pair"); _ints(pair_of_row, pairs, "pair_of_row")
    _ints(tiles, 3 * route_max_tiles(pairs, E, tile_rows), "expert tiles"); _ints(n_tiles, 1, "tile count")
    check(library().sp_route(_stream(), logits.data_ptr(), ids.data_ptr(), weights.data_ptr(), T, E, top, tile_rows,
                             row_of_pair.data_ptr(), pair_of_row.data_ptr(), tiles.data_ptr(), n_tiles.data_ptr()))


def route_sigmoid(logits: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, row_of_pair, pair_of_row, tiles, n_tiles,
                  tile_rows: int = 64) -> None:
    """`route` whose weights are the sigmoid of each chosen logit, not renormalised."""
    _gpu(logits, "router logits"); _gpu(ids, "chosen experts"); _gpu(weights, "expert weights")
    T, E = logits.shape
    top = ids.shape[1]
    if logits.dtype != torch.float32 or ids.dtype != torch.int32 or weights.dtype != torch.float32 or \
            tuple(ids.shape) != (T, top) or tuple(weights.shape) != (T, top) or not 0 < top <= E:
        raise KernelError("route_sigmoid: float32 logits [T, E], int32 ids and float32 weights [T, top] expected")
    pairs = T * top
    _ints(row_of_pair, pairs, "row_of_pair"); _ints(pair_of_row, pairs, "pair_of_row")
    _ints(tiles, 3 * route_max_tiles(pairs, E, tile_rows), "expert tiles"); _ints(n_tiles, 1, "tile count")
    check(library().sp_route_sigmoid(_stream(), logits.data_ptr(), ids.data_ptr(), weights.data_ptr(), T, E, top, tile_rows,
                                     row_of_pair.data_ptr(), pair_of_row.data_ptr(), tiles.data_ptr(), n_tiles.data_ptr()))


def route_sort(ids: torch.Tensor, experts: int, row_of_pair, pair_of_row, tiles, n_tiles, tile_rows: int = 64) -> None:
    """Orders the (token, choice) pairs by expert for the grouped products (see sprout_hip.h)."""
    pairs = ids.numel()
    _ints(ids, pairs, "chosen experts"); _ints(row_of_pair, pairs, "row_of_pair"); _ints(pair_of_row, pairs, "pair_of_row")
    _ints(tiles, 3 * route_max_tiles(pairs, experts, tile_rows), "expert tiles"); _ints(n_tiles, 1, "tile count")
    check(library().sp_route_sort(_stream(), ids.data_ptr(), pairs, experts, tile_rows, row_of_pair.data_ptr(),
                                  pair_of_row.data_ptr(), tiles.data_ptr(), n_tiles.data_ptr()))


def expert_gate_up(x: torch.Tensor, w: torch.Tensor, tiles, n_tiles, pair_of_row, top: int, out: torch.Tensor,
                   activation: str = "silu", tile_rows: int = 64, limit: float = 0.0) -> None:
    """out[row] = act(x[token] . w[e, :I]^T) * (x[token] . w[e, I:]^T) for every sorted row (w [experts, 2 I, K])."""
    _gpu(x, "expert input"); _gpu(w, "expert gate/up weights"); _gpu(out, "expert activations")
    T, K = x.shape
    E, two_i, _ = w.shape
    if w.shape[2] != K or two_i % 2 or tuple(out.shape) != (T * top, two_i // 2) or not (x.dtype == w.dtype == out.dtype):
        raise KernelError(f"expert_gate_up: shapes do not fit: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)}")
    max_tiles = route_max_tiles(T * top, E, tile_rows)
    _ints(tiles, 3 * max_tiles, "expert tiles"); _ints(n_tiles, 1, "tile count"); _ints(pair_of_row, T * top, "pair_of_row")
    check(library().sp_expert_gate_up(_stream(), _code(w, "expert weights"), x.data_ptr(), w.data_ptr(), tiles.data_ptr(),
                                      n_tiles.data_ptr(), max_tiles, tile_rows, pair_of_row.data_ptr(), top, out.data_ptr(),
                                      T, E, two_i // 2, K, variant_code(GATE_ACTIVATIONS, activation, "gate activation"),
                                      float(limit)))


def expert_down(act: torch.Tensor, w: torch.Tensor, tiles, n_tiles, out: torch.Tensor, tile_rows: int = 64) -> None:
    """out[row] (float32) = act[row] . w[e]^T for every sorted row (w [experts, hidden, I])."""
    _gpu(act, "expert activations"); _gpu(w, "expert down weights"); _gpu(out, "expert outputs")
    rows, inner = act.shape
    E, hidden, _ = w.shape
    if w.shape[2] != inner or tuple(out.shape) != (rows, hidden) or out.dtype != torch.float32 or act.dtype != w.dtype:
        raise KernelError(f"expert_down: shapes do not fit: act {tuple(act.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} {out.dtype}")
    max_tiles = route_max_tiles(rows, E, tile_rows)
    _ints(tiles, 3 * max_tiles, "expert tiles"); _ints(n_tiles, 1, "tile count")
    check(library().sp_expert_down(_stream(), _code(w, "expert weights"), act.data_ptr(), w.data_ptr(), tiles.data_ptr(),
                                   n_tiles.data_ptr(), max_tiles, tile_rows, out.data_ptr(), rows, E, hidden, inner))


def route_combine(y: torch.Tensor, row_of_pair, weights: torch.Tensor, residual: torch.Tensor, weighted: bool = True) -> None:
    """residual[t] += sum_k weights[t, k] * y[row_of_pair[t * top + k]]; with `weighted` False the rows are added as
    they are (`weights` then only says how many choices a token has)."""
    _gpu(y, "expert outputs"); _gpu(weights, "expert weights"); _gpu(residual, "residual")
    T, top = weights.shape
    H = residual.shape[1]
    if y.dtype != torch.float32 or tuple(y.shape) != (T * top, H) or residual.dtype != torch.float32 or residual.shape[0] < T \
            or weights.dtype != torch.float32:
        raise KernelError("route_combine: float32 outputs [T * top, H], weights [T, top] and residual [T, H] expected")
    _ints(row_of_pair, T * top, "row_of_pair")
    check(library().sp_route_combine(_stream(), y.data_ptr(), row_of_pair.data_ptr(), weights.data_ptr() if weighted else None,
                                     top, residual.data_ptr(), T, H))


def route_scored(logits: torch.Tensor, outputs: int, real: int, correction, groups: int, keep: int, scale: float,
                 ids: torch.Tensor, weights: torch.Tensor, row_of_pair, pair_of_row, tiles, n_tiles, tile_rows: int = 64) -> None:
    """Choice and order by another rule: scores = the softmax over the first `outputs` columns of a row of logits; the
    choice goes by score + correction and only inside the `keep` best of `groups` groups of neighbours; weights = the
    chosen scores times `scale`.  Outputs from `real` on are identity outputs: rows, but no tiles (see sprout_hip.h)."""
    _gpu(logits, "router logits"); _gpu(ids, "chosen experts"); _gpu(weights, "expert weights")
    T, stride = logits.shape
    top = ids.shape[1]
    if logits.dtype != torch.float32 or ids.dtype != torch.int32 or weights.dtype != torch.float32 or \
            tuple(ids.shape) != (T, top) or tuple(weights.shape) != (T, top) or not 0 < top <= outputs <= stride:
        raise KernelError("route_scored: float32 logits [T, >= outputs], int32 ids and float32 weights [T, top] expected")
    if correction is not None:
        _gpu(correction, "router correction")
        if correction.dtype != torch.float32 or correction.numel() != outputs:
            raise KernelError(f"route_scored: the correction must hold {outputs} float32 values")
    pairs = T * top
    _ints(row_of_pair, pairs, "row_of_pair"); _ints(pair_of_row, pairs, "pair_of_row")
    _ints(tiles, 3 * route_max_tiles(pairs, real, tile_rows), "expert tiles"); _ints(n_tiles, 1, "tile count")
    check(library().sp_route_scored(_stream(), logits.data_ptr(), stride, _ptr(correction), int(groups), int(keep), float(scale),
                                    ids.data_ptr(), weights.data_ptr(), T, outputs, real, top, tile_rows,
                                    row_of_pair.data_ptr(), pair_of_row.data_ptr(), tiles.data_ptr(), n_tiles.data_ptr()))


def route_combine_identity(y: torch.Tensor, row_of_pair, ids: torch.Tensor, weights: torch.Tensor, x: torch.Tensor, real: int,
                           residual: torch.Tensor) -> None:
    """residual[t] += sum_k weights[t, k] * (y[row_of_pair[t * top + k]] if ids[t, k] < real else x[t])."""
    _gpu(y, "expert outputs"); _gpu(weights, "expert weights"); _gpu(residual, "residual"); _gpu(x, "expert input")
    T, top = weights.shape
    H = residual.shape[1]
    if y.dtype != torch.float32 or tuple(y.shape) != (T * top, H) or residual.dtype != torch.float32 or residual.shape[0] < T \
            or weights.dtype != torch.float32 or x.shape[0] < T or x.shape[1] != H:
        raise KernelError("route_combine_identity: float32 outputs [T * top, H], weights [T, top], inputs and residual [T, H] expected")
    _ints(row_of_pair, T * top, "row_of_pair"); _ints(ids, T * top, "chosen experts")
    check(library().sp_route_combine_identity(_stream(), y.data_ptr(), row_of_pair.data_ptr(), weights.data_ptr(), top,
                                              ids.data_ptr(), _code(x, "expert input"), x.data_ptr(), int(real),
                                              residual.data_ptr(), T, H))


def qkv_prepare(proj: torch.Tensor, nq: int, nkv: int, dim: int, vdim: int, width: int, q_out: torch.Tensor, positions=None,
                inv_freq=None, inv_freq_tail=None, rotary_dim: int = 0, q_norm=None, k_norm=None, eps: float = 0.0,
                blend=None, first=None, keep_first: bool = False, slot_mapping=None, k_pool=None, v_pool=None,
                magnitude: float = 1.0, head_norm: bool = False) -> None:
    """From rows of projections [q | k | v] (heads of `dim`, `dim` and `vdim` numbers): optional RMS norm over the whole
    q row and the whole k row, optional rotation of the heads' first rotary_dim numbers, optional blend of the values
    with `first` (or `first` <- values), q to q_out [T, nq * width], k and v into pools that keep both `width` wide
    (zeros behind); cosines and sines times `magnitude`; with `head_norm` every q and k head is divided, after turning,
    by its root mean square over dim (`eps` inside the root); see sprout_hip.h."""
    _gpu(proj, "projections"); _gpu(q_out, "queries")
    T, stride = proj.shape
    if stride < (nq + nkv) * dim + nkv * vdim or tuple(q_out.shape) != (T, nq * width) or q_out.dtype != proj.dtype:
        raise KernelError(f"qkv_prepare: rows of {stride} and queries {tuple(q_out.shape)} {q_out.dtype} do not fit the head sizes")
    if (q_norm is None) != (k_norm is None):
        raise KernelError("qkv_prepare: queries and keys are normed together or not at all")
    if q_norm is not None:
        _gpu(q_norm, "query norm"); _gpu(k_norm, "key norm")
        if q_norm.dtype != proj.dtype or k_norm.dtype != proj.dtype or q_norm.numel() != nq * dim or k_norm.numel() != nkv * dim:
            raise KernelError("qkv_prepare: the norm weights must cover the whole q row and the whole k row")
    if rotary_dim:
        _ints(positions, T, "positions"); _gpu(inv_freq, "inv_freq")
        if inv_freq.dtype != torch.float32 or inv_freq.numel() < rotary_dim // 2 or rotary_dim % 2 or rotary_dim > dim:
            raise KernelError("qkv_prepare: inv_freq must hold rotary_dim / 2 float32 values, rotary_dim even and at most dim")
        if inv_freq_tail is not None and (inv_freq_tail.dtype != torch.float32 or inv_freq_tail.numel() != inv_freq.numel()):
            raise KernelError("qkv_prepare: inv_freq_tail must be float32 and as long as inv_freq")
    if blend is not None or keep_first:
        _gpu(first, "first values")
        if first.dtype != proj.dtype or first.shape[0] < T or first.shape[1] != nkv * vdim:
            raise KernelError(f"qkv_prepare: the first layer's values must be [>= {T}, {nkv * vdim}] {proj.dtype}")
        if blend is not None and (blend.dtype != proj.dtype or blend.numel() != 1 or not blend.is_cuda):
            raise KernelError("qkv_prepare: the blend factor is one number of the projections' dtype on the GPU")
    page_size = num_pages = 0
    if slot_mapping is not None:
        _ints(slot_mapping, T, "slot_mapping")
        num_pages, page_size = _check_pools(k_pool, v_pool, nkv, width, proj.dtype, "qkv_prepare")
    check(library().sp_qkv_prepare(_stream(), _code(proj, "projections"), proj.data_ptr(), stride, nq, nkv, dim, vdim, width,
                                   _ptr(q_norm), _ptr(k_norm), float(eps), _ptr(positions) if rotary_dim else None,
                                   _ptr(inv_freq) if rotary_dim else None, _ptr(inv_freq_tail) if rotary_dim else None,
                                   int(rotary_dim), _ptr(blend), _ptr(first), int(bool(keep_first)), _ptr(slot_mapping),
                                   _ptr(k_pool) if slot_mapping is not None else None,
                                   _ptr(v_pool) if slot_mapping is not None else None, page_size, num_pages, q_out.data_ptr(), T,
                                   float(magnitude), int(bool(head_norm))))


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
              workspace=None, kind: int = 0, project=None, scores: str = "scaled_dot", softcap: float = 0.0,
              sinks: torch.Tensor | None = None, mask_chunk: int | None = None, keep_first: int = 0) -> bool:
    """Causal attention of a mixed batch over paged keys and values (see sprout_hip.h).

    `workspace(n)` must return a float32 device tensor of at least n elements (default: a new one).
    `scores`: "scaled_dot", or "capped" (the scaled product s becomes softcap * tanh(s / softcap)).  `sinks`: float32
    [nq], one logit per query head that joins the softmax's denominator without a key or value.  `mask_chunk`: a
    query sees only the keys of its own block of that many positions, counted from position 0.
    `keep_first`: a sequence's first keep_first keys stay visible to every later query beside its `window`; the
    bfloat16 kernels and the float32-arithmetic kernel on the vector units know them, and such a call runs on those.
    `project`: (w_o [hidden, nq * hd], residual float32 [T, hidden]) of an output projection without bias
    that may be folded in: where the kernels take the step that way (one-query sequences only, bfloat16),
    residual += attention . w_o^T, `out` is left untouched and True is returned; otherwise False, and the
    projection is the caller's.
    """
    scores_code = variant_code(SCORE_STAGES, scores, "score stage")
    if scores_code == 1 and not softcap > 0.0:
        raise KernelError("attention: capped scores need a positive cap")
    if sinks is not None:
        _gpu(sinks, "sinks")
        if sinks.dtype != torch.float32 or sinks.numel() != nq:
            raise KernelError(f"attention: sinks must be {nq} float32 values")
    stage = (float(softcap), _ptr(sinks), int(mask_chunk) if mask_chunk else 0)
    keep_first = int(keep_first) if window else 0      # without a window every earlier key is visible anyway
    if keep_first < 0 or (keep_first and mask_chunk):
        raise KernelError("attention: kept first keys go with a window alone, and their number is not negative")
    if keep_first and (kind != 0 or q.dtype != torch.bfloat16):
        kind = 2      # the bfloat16 kernels know kept first keys; of the float32-arithmetic kernels the one on the vector units
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
                float(scale), scores_code, *stage))
            return True
    check(library().sp_attention(_stream(), _code(q, "q"), q.data_ptr(), q_stride, k_pool.data_ptr(), v_pool.data_ptr(),
                                 block_tables.data_ptr(), block_tables.shape[1], batch.q_start.data_ptr(),
                                 batch.q_len.data_ptr(), batch.ctx_len.data_ptr(), _ptr(tiles) if n_tiles else None,
                                 n_tiles, tile_q, max_tile_ctx, int(batch.mean_walk),
                                 _ptr(decode) if n_decode and decode is not None else None, n_decode,
                                 max_decode_ctx, _ptr(ws),
                                 need, out.data_ptr(), nq, nkv, hd, page_size, num_pages, int(window) if window else 0,
                                 float(scale), kind, scores_code, *stage, keep_first))
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


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor, out: torch.Tensor, inv_freq_tail=None,
               magnitude: float = 1.0) -> None:
    """out[t, d] = magnitude * (cos, sin) of positions[t] * inv_freq[d]; out float32 [T, len(inv_freq), 2].  With
    `inv_freq_tail` (what the float32 table lost of the exact one) angles, sines and cosines are taken in float64."""
    _gpu(inv_freq, "inv_freq"); _gpu(out, "rotation table")
    T, half = out.shape[0], inv_freq.numel()
    _ints(positions, T, "positions")
    if inv_freq.dtype != torch.float32 or out.dtype != torch.float32 or tuple(out.shape) != (T, half, 2):
        raise KernelError("rope_table: inv_freq float32 [half] and out float32 [T, half, 2] expected")
    if inv_freq_tail is not None:
        _gpu(inv_freq_tail, "inv_freq_tail")
        if inv_freq_tail.dtype != torch.float32 or inv_freq_tail.numel() != half:
            raise KernelError("rope_table: inv_freq_tail must be float32 and as long as inv_freq")
    check(library().sp_rope_table(_stream(), positions.data_ptr(), inv_freq.data_ptr(), _ptr(inv_freq_tail), half,
                                  float(magnitude), out.data_ptr(), T))


def scale(x: torch.Tensor, factor: float) -> None:
    """x *= factor, float32, in place."""
    _gpu(x, "scaled tensor")
    if x.dtype != torch.float32:
        raise KernelError("scale: float32 expected")
    check(library().sp_scale(_stream(), x.data_ptr(), float(factor), x.numel()))


def scaled_add(residual: torch.Tensor, a: torch.Tensor, scale_a: torch.Tensor, mult_a: float, b=None, scale_b=None,
               mult_b: float = 0.0) -> None:
    """residual [T, H] += mult_a * scale_a * a (+ mult_b * scale_b * b): float32 rows times learned vectors of H numbers."""
    _gpu(residual, "residual"); _gpu(a, "first summand"); _gpu(scale_a, "first scale")
    T, H = residual.shape
    if residual.dtype != torch.float32 or a.dtype != torch.float32 or a.shape[0] < T or a.shape[1] != H or scale_a.numel() != H:
        raise KernelError(f"scaled_add: residual {tuple(residual.shape)} {residual.dtype}, summand {tuple(a.shape)} {a.dtype}, "
                          f"scale of {scale_a.numel()} do not fit")
    if b is not None:
        _gpu(b, "second summand"); _gpu(scale_b, "second scale")
        if b.dtype != torch.float32 or b.shape[0] < T or b.shape[1] != H or scale_b.numel() != H or scale_b.dtype != scale_a.dtype:
            raise KernelError("scaled_add: the second summand does not fit the first")
    check(library().sp_scaled_add(_stream(), residual.data_ptr(), a.data_ptr(), _code(scale_a, "scale"), scale_a.data_ptr(),
                                  float(mult_a), _ptr(b), _ptr(scale_b) if b is not None else None, float(mult_b), T, H))


def head_gate(x: torch.Tensor, gate: torch.Tensor, gate_offset: int, heads: int, width: int) -> None:
    """x [T, heads * width] *= sigmoid(gate[t, gate_offset + head]), in place; x and gate of one dtype."""
    _gpu(x, "gated heads"); _gpu(gate, "head gate")
    T = x.shape[0]
    if x.shape[1] != heads * width or gate.dtype != x.dtype or gate.shape[0] < T or gate_offset < 0 or gate_offset + heads > gate.shape[1]:
        raise KernelError(f"head_gate: heads {tuple(x.shape)} {x.dtype} and gate {tuple(gate.shape)} {gate.dtype} do not fit")
    check(library().sp_head_gate(_stream(), _code(x, "gated heads"), x.data_ptr(), gate.data_ptr() + gate_offset * gate.element_size(),
                                 gate.shape[1], T, heads, width))


def rglru_takes(width: int, blocks: int, taps: int) -> bool:
    return bool(library().sp_rglru_takes(int(width), int(blocks), int(taps)))


def rglru(proj: torch.Tensor, y_off: int, x_off: int, width: int, blocks: int, taps: int, conv_w, conv_b, wa, ba, wi, bi, lam,
          q_start, q_len, seq_of_token, state_slots, n_seqs: int, state: torch.Tensor, tail, decay: torch.Tensor,
          drive: torch.Tensor, out: torch.Tensor, max_q_len: int = 0, workspace=None) -> None:
    """The gated linear recurrence of sp_rglru (sprout_hip.h) on a step's tokens.  `wa`, `wi`: [blocks, in, out].
    `max_q_len`: the most tokens one request brings (0: unknown); with `workspace(n)` (a float32 device tensor of at least
    n elements) long portions are walked in chunks side by side."""
    T, n = out.shape[0], width // max(blocks, 1)
    for t, what in ((proj, "projections"), (out, "recurrence output"), (state, "recurrent state"), (decay, "decay scratch"),
                    (drive, "drive scratch")):
        _gpu(t, what)
    if proj.shape[0] < T or out.dtype != proj.dtype or tuple(out.shape) != (T, width) or max(y_off, x_off) + width > proj.shape[1]:
        raise KernelError(f"rglru: projections {tuple(proj.shape)} {proj.dtype} and output {tuple(out.shape)} {out.dtype} do not fit")
    for t, shape, what in ((conv_w, (width, taps), "conv"), (conv_b, (width,), "conv bias"), (wa, (blocks, n, n), "gate matrices"),
                           (wi, (blocks, n, n), "gate matrices"), (ba, (blocks, n), "gate bias"), (bi, (blocks, n), "gate bias"),
                           (lam, (width,), "lam")):
        _gpu(t, what)
        if tuple(t.shape) != shape or t.dtype != proj.dtype:
            raise KernelError(f"rglru: {what} must be {shape} {proj.dtype}, got {tuple(t.shape)} {t.dtype}")
    for t, count, what in ((q_start, n_seqs, "q_start"), (q_len, n_seqs, "q_len"), (state_slots, n_seqs, "state_slots"),
                           (seq_of_token, T, "seq_of_token")):
        _ints(t, count, what)
    if state.dtype != torch.float32 or state.dim() != 2 or state.shape[1] != width:
        raise KernelError("rglru: the state must be float32 [slots, width]")
    if taps > 1:
        _gpu(tail, "convolution tail")
        if tail.dtype != torch.float32 or tuple(tail.shape) != (state.shape[0], taps - 1, width):
            raise KernelError("rglru: the convolution's kept inputs must be float32 [slots, taps - 1, width]")
    for t in (decay, drive):
        if t.dtype != torch.float32 or t.numel() < T * width:
            raise KernelError("rglru: scratch must hold float32 [T, width]")
    carry = None
    need = library().sp_rglru_carry_floats(width, n_seqs, int(max_q_len), T) if workspace is not None else 0
    if need:
        carry = workspace(need)
        if carry.dtype != torch.float32 or carry.numel() < need or not carry.is_cuda:
            raise KernelError("rglru: workspace too small")
    check(library().sp_rglru(_stream(), _code(proj, "projections"), proj.data_ptr(), proj.shape[1], y_off, x_off, width, blocks,
                             taps, conv_w.data_ptr(), conv_b.data_ptr(), wa.data_ptr(), ba.data_ptr(), wi.data_ptr(), bi.data_ptr(),
                             lam.data_ptr(), q_start.data_ptr(), q_len.data_ptr(), seq_of_token.data_ptr(), state_slots.data_ptr(),
                             state.data_ptr(), _ptr(tail) if taps > 1 else None, decay.data_ptr(), drive.data_ptr(),
                             out.data_ptr(), T, n_seqs, int(max_q_len) if carry is not None else 0, _ptr(carry)))


def _step_ints(q_start, q_len, state_slots, n_seqs: int, seq_of_token=None, T: int = 0) -> None:
    for t, what in ((q_start, "q_start"), (q_len, "q_len"), (state_slots, "state_slots")):
        _ints(t, n_seqs, what)
    if seq_of_token is not None:
        _ints(seq_of_token, T, "seq_of_token")


def short_conv(x: torch.Tensor, x_off: int, channels: int, taps: int, w: torch.Tensor, bias, out: torch.Tensor, out_off: int,
               q_start, q_len, seq_of_token, state_slots, n_seqs: int, state, act: str | None = None,
               add_input: bool = False, max_q_len: int = 0) -> None:
    """The causal convolution of sp_short_conv (sprout_hip.h) on columns x_off .. x_off + channels of a step's rows `x`, into
    columns out_off .. of `out` (another tensor of the same dtype).  `w`: TAP-major [taps, channels].  `state`: float32
    [slots, taps - 1, channels], the requests' last inputs, read and left behind; None with one tap.  `act`: None or
    "silu".  `max_q_len`: the most tokens one request brings (0: unknown)."""
    _gpu(x, "convolution input"); _gpu(out, "convolution output"); _gpu(w, "convolution weights")
    T = out.shape[0]
    if x.dim() != 2 or out.dim() != 2 or x.shape[0] < T or x.dtype != out.dtype or x_off + channels > x.shape[1] \
            or out_off + channels > out.shape[1] or x.data_ptr() == out.data_ptr():
        raise KernelError(f"short_conv: rows {tuple(x.shape)} {x.dtype} and {tuple(out.shape)} {out.dtype} do not fit {channels} channels")
    if tuple(w.shape) != (taps, channels) or not w.is_contiguous() or (bias is not None and (bias.numel() != channels or bias.dtype != w.dtype)):
        raise KernelError(f"short_conv: weights must be tap-major [{taps}, {channels}] with a bias of {channels}")
    if act not in (None, "silu"):
        raise KernelError(f"short_conv: no activation {act!r}")
    _step_ints(q_start, q_len, state_slots, n_seqs, seq_of_token, T)
    if taps > 1:
        _gpu(state, "convolution state")
        if state.dtype != torch.float32 or state.dim() != 3 or tuple(state.shape[1:]) != (taps - 1, channels) or not state.is_contiguous():
            raise KernelError(f"short_conv: the state must be float32 [slots, {taps - 1}, {channels}]")
    if bias is not None:
        _gpu(bias, "convolution bias")
    check(library().sp_short_conv(_stream(), _code(x, "convolution input"), x.data_ptr(), x.stride(0), x_off, channels, taps,
                                  _code(w, "convolution weights"), w.data_ptr(), _ptr(bias), 1 if act == "silu" else 0,
                                  int(bool(add_input)), out.data_ptr(), out.stride(0), out_off, q_start.data_ptr(),
                                  q_len.data_ptr(), seq_of_token.data_ptr(), state_slots.data_ptr(),
                                  state.data_ptr() if taps > 1 else None, T, n_seqs, int(max_q_len)))


def group_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: torch.Tensor, parts: int) -> None:
    """out = x / sqrt(mean(x^2) + eps) * weight with the mean over each of a row's `parts` equal parts; x float32 [T, n]."""
    _gpu(x, "norm input"); _gpu(weight, "norm weight"); _gpu(out, "norm output")
    T, n = out.shape
    if x.dtype != torch.float32 or tuple(x.shape) != (T, n) or weight.numel() != n or parts <= 0 or n % parts \
            or not x.is_contiguous() or not out.is_contiguous():
        raise KernelError(f"group_rmsnorm: float32 rows {tuple(x.shape)}, weight {tuple(weight.shape)} and {parts} parts do not fit")
    check(library().sp_group_rmsnorm(_stream(), x.data_ptr(), _code(weight, "norm weight"), weight.data_ptr(), float(eps),
                                     _code(out, "norm output"), out.data_ptr(), T, parts, n // parts))


UNARY_ACTIVATIONS = {"gelu_erf": 0}      # x * Phi(x), the exact GELU


def activation(x: torch.Tensor, kind: str) -> None:
    """In place: x <- act(x), `kind` one of UNARY_ACTIVATIONS."""
    _gpu(x, "activation input")
    if not x.is_contiguous():
        raise KernelError("activation: rows must be contiguous")
    check(library().sp_activation(_stream(), _code(x, "activation input"), x.data_ptr(), x.numel(),
                                  variant_code(UNARY_ACTIVATIONS, kind, "activation")))


def scale_rows(x: torch.Tensor, weights: torch.Tensor, out: torch.Tensor) -> None:
    """out[t * top + k] = x[t] * weights[t, k]: a token's row once per choice, times the choice's weight."""
    _gpu(x, "rows"); _gpu(weights, "row weights"); _gpu(out, "scaled rows")
    T, top = weights.shape
    H = x.shape[1]
    if weights.dtype != torch.float32 or x.shape[0] < T or tuple(out.shape) != (T * top, H) or out.dtype != x.dtype \
            or not x.is_contiguous() or not out.is_contiguous():
        raise KernelError("scale_rows: rows [T, H], float32 weights [T, top] and an output [T * top, H] of the rows' dtype expected")
    check(library().sp_scale_rows(_stream(), _code(x, "rows"), x.data_ptr(), weights.data_ptr(), top, out.data_ptr(), T, H))


def _scan_scratch(need: int, workspace):
    """The scratch of a scan that walks long portions in chunks: None where the step needs none or the caller has none."""
    if not need or workspace is None:
        return None
    scratch = workspace(need)
    if scratch.dtype != torch.float32 or scratch.numel() < need or not scratch.is_cuda:
        raise KernelError("scan: workspace too small")
    return scratch


def ssd_scan(proj: torch.Tensor, z_off: int, dt_off: int, xbc: torch.Tensor, heads: int, vdim: int, state_size: int, groups: int,
             dt_bias, a_log, skip, q_start, q_len, state_slots, n_seqs: int, state: torch.Tensor, out: torch.Tensor,
             max_q_len: int = 0, workspace=None) -> None:
    """The state-space-duality scan of sp_ssd_scan (sprout_hip.h); out float32 [T, heads * vdim] = y * silu(z).
    `max_q_len`: the most tokens one request brings (0: unknown); with `workspace(n)` (a float32 device tensor of at least
    n elements) long portions are walked in chunks side by side."""
    for t, what in ((proj, "projections"), (xbc, "convolved rows"), (state, "state"), (out, "scan output")):
        _gpu(t, what)
    T, inner = out.shape[0], heads * vdim
    if proj.shape[0] < T or xbc.shape[0] < T or proj.dtype != xbc.dtype or out.dtype != torch.float32 or tuple(out.shape) != (T, inner) \
            or not out.is_contiguous():
        raise KernelError("ssd_scan: rows and output do not fit")
    for t in (dt_bias, a_log, skip):
        _gpu(t, "head constants")
        if t.dtype != torch.float32 or t.numel() != heads:
            raise KernelError(f"ssd_scan: one float32 constant per head ({heads}) expected")
    if state.dtype != torch.float32 or tuple(state.shape[1:]) != (heads, state_size, vdim) or not state.is_contiguous():
        raise KernelError(f"ssd_scan: the state must be float32 [slots, {heads}, {state_size}, {vdim}]")
    _step_ints(q_start, q_len, state_slots, n_seqs)
    scratch = _scan_scratch(library().sp_ssd_scan_scratch_floats(heads, vdim, state_size, n_seqs, int(max_q_len)), workspace)
    check(library().sp_ssd_scan(_stream(), _code(proj, "projections"), proj.data_ptr(), proj.stride(0), z_off, dt_off,
                                xbc.data_ptr(), xbc.stride(0), heads, vdim, state_size, groups, dt_bias.data_ptr(),
                                a_log.data_ptr(), skip.data_ptr(), q_start.data_ptr(), q_len.data_ptr(), state_slots.data_ptr(),
                                state.data_ptr(), out.data_ptr(), T, n_seqs, int(max_q_len) if scratch is not None else 0,
                                _ptr(scratch)))


def selective_scan(u: torch.Tensor, u_off: int, z: torch.Tensor, z_off: int, dt: torch.Tensor, bc: torch.Tensor, bc_off: int,
                   inner: int, state_size: int, a, skip, q_start, q_len, state_slots, n_seqs: int, state: torch.Tensor,
                   out: torch.Tensor, max_q_len: int = 0, workspace=None) -> None:
    """The selective scan of sp_selective_scan (sprout_hip.h); out [T, inner] of the rows' dtype = y * silu(z).
    `max_q_len`, `workspace`: as for ssd_scan."""
    for t, what in ((u, "inputs"), (z, "gates"), (dt, "step sizes"), (bc, "B and C"), (state, "state"), (out, "scan output")):
        _gpu(t, what)
    T = out.shape[0]
    if min(u.shape[0], z.shape[0], dt.shape[0], bc.shape[0]) < T or not (u.dtype == z.dtype == bc.dtype == out.dtype) \
            or dt.dtype != torch.float32 or tuple(dt.shape[1:]) != (inner,) or tuple(out.shape) != (T, inner) \
            or not dt.is_contiguous() or not out.is_contiguous():
        raise KernelError("selective_scan: rows and output do not fit")
    _gpu(a, "decay rates"); _gpu(skip, "skip weights")
    if a.dtype != torch.float32 or tuple(a.shape) != (inner, state_size) or skip.dtype != torch.float32 or skip.numel() != inner:
        raise KernelError(f"selective_scan: float32 rates [{inner}, {state_size}] and skips [{inner}] expected")
    if state.dtype != torch.float32 or tuple(state.shape[1:]) != (inner, state_size) or not state.is_contiguous():
        raise KernelError(f"selective_scan: the state must be float32 [slots, {inner}, {state_size}]")
    _step_ints(q_start, q_len, state_slots, n_seqs)
    scratch = _scan_scratch(library().sp_selective_scan_scratch_floats(inner, state_size, n_seqs, int(max_q_len)), workspace)
    check(library().sp_selective_scan(_stream(), _code(u, "inputs"), u.data_ptr(), u.stride(0), u_off, z.data_ptr(), z.stride(0),
                                      z_off, dt.data_ptr(), bc.data_ptr(), bc.stride(0), bc_off, inner, state_size, a.data_ptr(),
                                      skip.data_ptr(), q_start.data_ptr(), q_len.data_ptr(), state_slots.data_ptr(),
                                      state.data_ptr(), out.data_ptr(), T, n_seqs, int(max_q_len) if scratch is not None else 0,
                                      _ptr(scratch)))


def qk_cross_prepare(qk: torch.Tensor, nq: int, nkv: int, dim: int, width: int, q_norm, k_norm, eps: float, positions, freq,
                     rotary_dim: int, q_out: torch.Tensor, slot_mapping=None, k_pool=None, v_pool=None) -> None:
    """sp_qk_cross_prepare (sprout_hip.h): head norms, turning in neighbouring pairs, and the (query head, value head)
    pairs as heads of their own: queries to q_out [T, nq * nkv * width], keys and values into pools of nkv * nkv heads."""
    _gpu(qk, "q and k rows"); _gpu(q_out, "prepared queries"); _gpu(q_norm, "q norm"); _gpu(k_norm, "k norm")
    T = q_out.shape[0]
    if qk.shape[0] < T or qk.shape[1] != (nq + nkv) * dim or not qk.is_contiguous() or q_out.dtype != qk.dtype \
            or tuple(q_out.shape) != (T, nq * nkv * width) or not q_out.is_contiguous():
        raise KernelError(f"qk_cross_prepare: rows {tuple(qk.shape)} and queries {tuple(q_out.shape)} do not fit")
    if q_norm.numel() != dim or k_norm.numel() != dim or q_norm.dtype != k_norm.dtype:
        raise KernelError(f"qk_cross_prepare: norm weights of {dim} numbers expected")
    _ints(positions, T, "positions")
    if rotary_dim:
        _gpu(freq, "frequencies")
        if freq.dtype != torch.float64 or freq.numel() < rotary_dim // 2:
            raise KernelError("qk_cross_prepare: a float64 table of one frequency per pair expected")
    page_size = 0
    if slot_mapping is not None:
        _ints(slot_mapping, T, "slot_mapping")
        _, page_size = _check_pools(k_pool, v_pool, nkv * nkv, width, qk.dtype, "qk_cross_prepare")
    check(library().sp_qk_cross_prepare(_stream(), _code(qk, "q and k rows"), qk.data_ptr(), nq, nkv, dim, width,
                                        _code(q_norm, "q norm"), q_norm.data_ptr(), k_norm.data_ptr(), float(eps),
                                        positions.data_ptr(), _ptr(freq) if rotary_dim else None, rotary_dim, _ptr(slot_mapping),
                                        q_out.data_ptr(), _ptr(k_pool), _ptr(v_pool), page_size, T))


def head_mix(o: torch.Tensor, talk: torch.Tensor, nq: int, nkv: int, dim: int, width: int, out: torch.Tensor) -> None:
    """sp_head_mix (sprout_hip.h): the outputs of the (query head, value head) heads mixed by `talk` float32 [nq, nq]."""
    _gpu(o, "attention outputs"); _gpu(talk, "head mixing matrix"); _gpu(out, "mixed heads")
    T = out.shape[0]
    if o.shape[0] < T or o.shape[1] != nq * nkv * width or not o.is_contiguous() or out.dtype != o.dtype \
            or tuple(out.shape) != (T, nq * dim) or not out.is_contiguous() or talk.dtype != torch.float32 \
            or tuple(talk.shape) != (nq, nq) or not talk.is_contiguous():
        raise KernelError("head_mix: outputs, matrix and result do not fit")
    check(library().sp_head_mix(_stream(), _code(o, "attention outputs"), o.data_ptr(), talk.data_ptr(), nq, nkv, dim, width,
                                out.data_ptr(), T))


def retention_takes(dim: int, vdim: int) -> bool:
    return bool(library().sp_retention_takes(int(dim), int(vdim)))


def retention(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, g_off: int, heads: int, dim: int, vdim: int,
              rotary_dim: int, cos_sin, decay: torch.Tensor, eps: float, q_start, q_len, state_slots, n_seqs: int,
              state: torch.Tensor, out: torch.Tensor, max_q_len: int = 0, workspace=None) -> None:
    """Retention of sp_retention (sprout_hip.h) on a step's tokens; `cos_sin`: rope_table of the step's positions.
    `max_q_len`, `workspace`: as for `rglru`."""
    T = out.shape[0]
    _gpu(proj, "projections"); _gpu(out, "retention output"); _gpu(state, "retention state"); _gpu(decay, "decays")
    if proj.shape[0] < T or out.dtype != proj.dtype or tuple(out.shape) != (T, heads * vdim):
        raise KernelError(f"retention: projections {tuple(proj.shape)} {proj.dtype} and output {tuple(out.shape)} {out.dtype} do not fit")
    if max(q_off, k_off) + heads * dim > proj.shape[1] or max(v_off, g_off) + heads * vdim > proj.shape[1] or min(q_off, k_off, v_off, g_off) < 0:
        raise KernelError("retention: a row of projections does not hold q, k, v and the gate")
    if decay.dtype != torch.float32 or decay.numel() != heads:
        raise KernelError(f"retention: decays must be {heads} float32 values")
    if state.dtype != torch.float32 or tuple(state.shape[1:]) != (heads, dim, vdim):
        raise KernelError(f"retention: the state must be float32 [slots, {heads}, {dim}, {vdim}]")
    if rotary_dim:
        _gpu(cos_sin, "rotation table")
        if cos_sin.dtype != torch.float32 or cos_sin.shape[0] < T or tuple(cos_sin.shape[1:]) != (rotary_dim // 2, 2):
            raise KernelError("retention: the rotation table must be float32 [T, rotary_dim / 2, 2]")
    for t, what in ((q_start, "q_start"), (q_len, "q_len"), (state_slots, "state_slots")):
        _ints(t, n_seqs, what)
    scratch = None
    need = library().sp_retention_scratch_floats(heads, dim, vdim, n_seqs, int(max_q_len), T) if workspace is not None else 0
    if need:
        scratch = workspace(need)
        if scratch.dtype != torch.float32 or scratch.numel() < need or not scratch.is_cuda:
            raise KernelError("retention: workspace too small")
    check(library().sp_retention(_stream(), _code(proj, "projections"), proj.data_ptr(), proj.shape[1], q_off, k_off, v_off, g_off,
                                 heads, dim, vdim, rotary_dim, _ptr(cos_sin) if rotary_dim else None, decay.data_ptr(), float(eps),
                                 q_start.data_ptr(), q_len.data_ptr(), state_slots.data_ptr(), state.data_ptr(), out.data_ptr(),
                                 T, n_seqs, int(max_q_len) if scratch is not None else 0, _ptr(scratch)))


def gemm_from_residual(residual: torch.Tensor, norm_weight: torch.Tensor, eps: float, w: torch.Tensor, out: torch.Tensor,
                       bias: torch.Tensor | None = None) -> bool:
    """out (bfloat16 [T, N]) = (rmsnorm(residual) * norm_weight) . w^T (+ bias) in one kernel, for the few tokens of a decode
    step: the norm is the product's prologue.  Returns False (and does nothing) where the kernel does not take the shape
    or a norm kernel before the product would be faster; the caller then norms and multiplies in turn."""
    N, K = w.shape
    T = residual.shape[0]
    if (w.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or tuple(out.shape) != (T, N) or T > 64
            or not fused_supported(0, T, N, K, norm=True) or not fused_norm_pays(T, N, K)):
        return False
    _gpu(w, "weight"); _gpu(out, "output")
    xp, rp, nd, npt, _ = _activations(None, residual, norm_weight, K, "gemm_from_residual")
    if bias is not None:
        _gpu(bias, "bias")
        if bias.numel() != N:
            raise KernelError(f"gemm_from_residual: bias has {bias.numel()} values for {N} columns")
    check(library().sp_gemm_decode(_stream(), xp, rp, nd, npt, float(eps), w.data_ptr(), _code(bias, "bias") if bias is not None else 0,
                                   _ptr(bias), STORE, out.data_ptr(), T, N, K))
    return True


def gate_up_silu(w: torch.Tensor, out: torch.Tensor, x=None, residual=None, norm_weight=None, eps: float = 0.0,
                 activation: str = "silu", limit: float = 0.0, row_gate=None, row_gate_column: int = 0) -> None:
    """out = act(a . w[:I]^T, a . w[I:]^T) for activations a as in `qkv_rope_cache`, times sigmoid(row_gate[t, column])
    where row_gate (float32 [T, columns]) is given."""
    _gpu(w, "gate/up weight"); _gpu(out, "gated output")
    N, K = w.shape
    xp, rp, nd, npt, T = _activations(x, residual, norm_weight, K, "gate_up_silu")
    if w.dtype != torch.bfloat16 or N % 2 or tuple(out.shape) != (T, N // 2) or out.dtype != torch.bfloat16:
        raise KernelError("gate_up_silu: weight [2 I, K] and output [T, I] bfloat16 expected")
    check(library().sp_gate_up_silu(_stream(), xp, rp, nd, npt, float(eps), w.data_ptr(), out.data_ptr(), T, N // 2, K,
                                    variant_code(GATE_ACTIVATIONS, activation, "gate activation"), float(limit),
                                    *_row_gate(row_gate, row_gate_column, T, "gate_up_silu")))


def gate_up_silu_f32(w: torch.Tensor, x: torch.Tensor, out: torch.Tensor, activation: str = "silu", norm_weight=None,
                     eps: float = 0.0, limit: float = 0.0, row_gate=None, row_gate_column: int = 0) -> bool:
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
                                        T, I, K, variant_code(GATE_ACTIVATIONS, activation, "gate activation"), float(limit),
                                        *_row_gate(row_gate, row_gate_column, T, "gate_up_silu_f32")))
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


def _row_gate(row_gate, column: int, T: int, what: str):
    """(pointer, stride) of a float32 [>= T, columns] tensor's column, or (None, 0)."""
    if row_gate is None:
        return None, 0
    _gpu(row_gate, "row gate")
    if row_gate.dtype != torch.float32 or row_gate.dim() != 2 or row_gate.shape[0] < T or not 0 <= column < row_gate.shape[1]:
        raise KernelError(f"{what}: the row gate must be float32 [>= T, columns]")
    return row_gate.data_ptr() + 4 * column, row_gate.shape[1]


def silu_mul(gu: torch.Tensor, out: torch.Tensor, activation: str = "silu", limit: float = 0.0,
             row_gate: torch.Tensor | None = None, row_gate_column: int = 0) -> None:
    """out[t, i] = act(gu[t, i], gu[t, I + i]), times sigmoid(row_gate[t, row_gate_column]) where row_gate (float32
    [T, *]) is given."""
    _gpu(gu, "gate/up"); _gpu(out, "gated output")
    T, I = out.shape
    if tuple(gu.shape) != (T, 2 * I) or gu.dtype != out.dtype:
        raise KernelError(f"silu_mul: shapes do not fit: gu {tuple(gu.shape)}, out {tuple(out.shape)}")
    gate_ptr, gate_stride = _row_gate(row_gate, row_gate_column, T, "silu_mul")
    check(library().sp_silu_mul(_stream(), _code(gu, "gate/up"), gu.data_ptr(), out.data_ptr(), T, I,
                                variant_code(GATE_ACTIVATIONS, activation, "gate activation"), float(limit), gate_ptr, gate_stride))


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
