"""Checked Python entry points of the HIP kernels.

Every function checks on the host that operand shapes, types and strides are
what its kernel and grid assume, then launches on torch's current stream.
Tensors are torch CUDA tensors used as plain device memory; nothing here falls
back to a library routine.
"""
from __future__ import annotations

import torch

from .lib import library, check

F32, BF16 = 0, 1
_DTYPE_ID = {torch.float32: F32, torch.bfloat16: BF16}


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _need(cond, text):
    if not cond:
        raise ValueError(text)


def _dev(t, dtype=None, name="tensor"):
    _need(isinstance(t, torch.Tensor) and t.is_cuda, f"{name} must be a CUDA tensor")
    if dtype is not None:
        _need(t.dtype == dtype, f"{name} must be {dtype}, is {t.dtype}")
    return t.data_ptr()


def _rows(t, name):
    """(rows, cols, leading dimension) of a 2-D tensor whose rows are contiguous."""
    _need(t.dim() == 2 and (t.shape[1] == 1 or t.stride(1) == 1), f"{name} must be 2-D with contiguous rows")
    ld = t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])
    _need(ld >= t.shape[1], f"{name} has overlapping rows")
    return t.shape[0], t.shape[1], ld


def dtype_id(dtype):
    _need(dtype in _DTYPE_ID, f"unsupported dtype {dtype}; float32 and bfloat16 are built")
    return _DTYPE_ID[dtype]


def probe_read(buffer, out, blocks=2048):
    """Launch the plain streaming reader over BUFFER (any contiguous device tensor); returns the bytes it reads.
    A yardstick for benchmarks: time it to get the device's own read ceiling."""
    import ctypes
    _need(buffer.is_contiguous(), "probe_read needs a contiguous buffer")
    n = ctypes.c_long(0)
    check(library().tw_probe_read(_dev(buffer), buffer.numel() * buffer.element_size(), _dev(out, torch.float32, "out"),
                                  int(blocks), ctypes.byref(n), _stream()), "probe_read")
    return int(n.value)


def upload_words(src, dst, segments):
    """dst[o:o + n] = src[o:o + n] for every (o, n) of SEGMENTS (at most 16), by a kernel on the current stream.

    src: a pinned int32 host tensor; dst: an int32 device tensor of the same length. A step's metadata goes to
    the device this way: a copy through the copy engine leaves the compute queue idle around it for tens of
    microseconds, a kernel that reads the pinned memory does not leave the queue."""
    import ctypes
    _need(src.dtype == torch.int32 and dst.dtype == torch.int32 and src.is_contiguous() and dst.is_contiguous(),
          "upload_words moves contiguous int32 buffers")
    _need(src.is_pinned() and dst.is_cuda and src.numel() == dst.numel(), "upload_words: pinned host words to as many device words")
    segments = [(int(o), int(n)) for o, n in segments if n > 0]
    _need(len(segments) <= 16 and all(o >= 0 and o + n <= dst.numel() for o, n in segments), "upload_words: bad segments")
    offsets = (ctypes.c_int * 16)(*[o for o, _ in segments])
    counts = (ctypes.c_int * 16)(*[n for _, n in segments])
    check(library().tw_upload_words(src.data_ptr(), dst.data_ptr(), len(segments), offsets, counts, _stream()), "upload_words")


def embed_gather(ids, table, out, feed=None):
    """out[n, :] = float32(table[ids[n], :]); an id -1 - k stands for feed[k] (int32, on the device)."""
    n = ids.numel()
    vocab, hidden = table.shape
    _need(table.is_contiguous() and out.is_contiguous(), "embedding operands must be contiguous")
    _need(tuple(out.shape) == (n, hidden), "embedding output has the wrong shape")
    check(library().tw_embed_gather(dtype_id(table.dtype), _dev(ids, torch.int32, "ids"), _dev(table),
                                    _dev(out, torch.float32, "out"), n, hidden, vocab,
                                    _dev(feed, torch.int32, "feed") if feed is not None else None,
                                    feed.numel() if feed is not None else 0, _stream()),
          "embed_gather")
    return out


def rmsnorm(x, weight, eps, out, rows=None, add=None, row_scratch=None):
    """out = x * rsqrt(mean(x^2) + eps) * weight per row; x float32, weight float32.

    rows: int32 indices choosing the input row of each output row.
    add: float32 [splits, n, hidden] partial sums first added to x. Without `rows`
    x itself is updated; with `rows` the sums go to row_scratch [n_out, hidden].
    """
    _need(x.dim() == 2 and x.is_contiguous(), "rmsnorm input must be contiguous [n, hidden]")
    n, hidden = x.shape
    n_out = rows.numel() if rows is not None else n
    _need(out.is_contiguous() and tuple(out.shape) == (n_out, hidden), "rmsnorm output has the wrong shape")
    _need(weight.numel() == hidden, "rmsnorm weight has the wrong size")
    add_ptr, splits, stride = None, 0, 0
    scratch_ptr = None
    if add is not None:
        _need(add.dim() == 3 and add.is_contiguous() and tuple(add.shape[1:]) == (n, hidden),
              "rmsnorm partial sums must be [splits, n, hidden]")
        add_ptr, splits, stride = _dev(add, torch.float32, "add"), add.shape[0], n * hidden
        if rows is not None:
            _need(row_scratch is not None and row_scratch.is_contiguous()
                  and tuple(row_scratch.shape) == (n_out, hidden), "rmsnorm with rows and partial sums needs row_scratch [n_out, hidden]")
            scratch_ptr = _dev(row_scratch, torch.float32, "row_scratch")
    check(library().tw_rmsnorm(dtype_id(out.dtype), _dev(x, torch.float32, "x"),
                               _dev(weight, torch.float32, "weight"), _dev(out),
                               _dev(rows, torch.int32, "rows") if rows is not None else None,
                               n_out, hidden, float(eps), add_ptr, splits, stride, scratch_ptr, _stream()), "rmsnorm")
    return out


def rope_table(positions, inv_freq, cos, sin, magnitude=1.0):
    """cos/sin[n, j] of float32(positions[n]) * inv_freq[j], both times MAGNITUDE."""
    n, half = positions.numel(), inv_freq.numel()
    _need(cos.is_contiguous() and sin.is_contiguous() and tuple(cos.shape) == (n, half)
          and tuple(sin.shape) == (n, half), "rotary tables must be [n, rot/2]")
    check(library().tw_rope_table(_dev(positions, torch.int32, "positions"),
                                  _dev(inv_freq, torch.float32, "inv_freq"),
                                  _dev(cos, torch.float32, "cos"), _dev(sin, torch.float32, "sin"),
                                  n, half, float(magnitude), _stream()), "rope_table")


def rope_kv_write(qkv, cos, sin, slots, keys, values, q_heads, kv_heads, head_dim, page_size,
                  write_cache=True, partial=None, bias=None, adjacent=False):
    """Rotate q (in place) and k of qkv[n] = [q | k | v]; write rotated k and v to the pages.

    Pair j of a head is elements (j, j + rot/2), or with `adjacent` elements (2j, 2j + 1).

    keys [pages, kv_heads, page_size, head_dim]; values hold the same number of
    elements and are written as [pages, kv_heads, head_dim, page_size].
    partial: float32 [splits, n, width] split-K sums of the projection; qkv is then
    first filled with round(sum of the splits + bias).
    """
    n, width, ld = _rows(qkv, "qkv")
    _need(width == (q_heads + 2 * kv_heads) * head_dim, "qkv width does not match the head counts")
    half = cos.shape[1] if cos is not None else 0
    rot = 2 * half
    _need(rot <= head_dim, "rotary dimension exceeds head_dim")
    if rot:
        _need(tuple(cos.shape) == (n, half) and tuple(sin.shape) == (n, half) and cos.is_contiguous()
              and sin.is_contiguous(), "rotary tables must be [n, rot/2]")
    if write_cache:
        _need(keys.dtype == qkv.dtype and values.dtype == qkv.dtype, "cache and qkv types differ")
        _need(keys.is_contiguous() and values.is_contiguous(), "cache tensors must be contiguous")
        _need(tuple(keys.shape[1:]) == (kv_heads, page_size, head_dim), "keys must be [pages, kv_heads, page_size, head_dim]")
        _need(values.numel() == keys.numel(), "keys and values differ in size")
        _need(slots.numel() == n, "one cache slot per token is needed")
    if partial is not None:
        _need(partial.dim() == 3 and partial.is_contiguous() and tuple(partial.shape[1:]) == (n, width),
              "projection partial sums must be [splits, n, width]")
        _need(bias is None or bias.numel() == width, "bias has the wrong size")
    dummy = qkv
    check(library().tw_rope_kv_write(
        dtype_id(qkv.dtype), _dev(qkv), ld,
        _dev(cos, torch.float32, "cos") if rot else _dev(dummy), _dev(sin, torch.float32, "sin") if rot else _dev(dummy),
        _dev(slots, torch.int32, "slots") if write_cache else None,
        _dev(keys) if write_cache else None, _dev(values) if write_cache else None,
        n, q_heads, kv_heads, head_dim, rot, page_size, 1 if write_cache else 0,
        _dev(partial, torch.float32, "partial") if partial is not None else None,
        partial.shape[0] if partial is not None else 0,
        _dev(bias, torch.float32, "bias") if (partial is not None and bias is not None) else None,
        1 if adjacent else 0, _stream()), "rope_kv_write")


def silu_mul(gate_up, out):
    """out[n, i] = silu(gate_up[n, i]) * gate_up[n, inter + i]."""
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 2 == 0, "gate_up must be contiguous [n, 2*inter]")
    n, inter = gate_up.shape[0], gate_up.shape[1] // 2
    _need(out.is_contiguous() and tuple(out.shape) == (n, inter) and out.dtype == gate_up.dtype,
          "silu_mul output has the wrong shape or type")
    check(library().tw_silu_mul(dtype_id(gate_up.dtype), _dev(gate_up), _dev(out), n, inter, _stream()), "silu_mul")
    return out


class ShuffledWeight:
    """An [n, k] weight in the kernels' own layout: an exact permutation of the matrix, zero padded.

    Blocks of 16 rows x 4 sixteen-byte chunks, stored in the order MFMA fragments are read:
    [ceil(n/16)][k_steps][chunk 0..3][row 0..15][elements of 16 bytes]. One wave-wide load of a
    block is 1 KB of consecutive memory.
    """

    def __init__(self, data, n, k, k_steps, dtype):
        self.data, self.n, self.k, self.k_steps, self.dtype = data, n, k, k_steps, dtype

    @property
    def shape(self):
        return (self.n, self.k)

    def numel(self):
        return self.data.numel()

    def element_size(self):
        return self.data.element_size()

    def to_rows(self):
        """The matrix back in row-major order (for tests)."""
        epf = 16 // self.data.element_size()
        blocks = self.data.view(-1, self.k_steps, 4, 16, epf)
        return blocks.permute(0, 3, 1, 2, 4).reshape(blocks.shape[0] * 16, self.k_steps * 4 * epf)[:self.n, :self.k]


def can_shuffle(weight):
    return weight.dim() == 2 and weight.shape[1] % (16 // weight.element_size()) == 0


def shuffle_weight(weight):
    """The shuffled copy of a row-major [n, k] weight (k must be a multiple of 16 bytes)."""
    _need(can_shuffle(weight), "only weights whose rows are a multiple of 16 bytes can be shuffled")
    n, k = weight.shape
    epf = 16 // weight.element_size()
    k_steps = (k // epf + 3) // 4
    n_pad, k_pad = (n + 15) // 16 * 16, k_steps * 4 * epf
    if (n_pad, k_pad) != (n, k):
        padded = weight.new_zeros((n_pad, k_pad))
        padded[:n, :k] = weight
    else:
        padded = weight
    data = padded.view(n_pad // 16, 16, k_steps, 4, epf).permute(0, 2, 3, 1, 4).contiguous().view(-1)
    return ShuffledWeight(data, n, k, k_steps, weight.dtype)


def _weight_args(weight):
    """(n, k, pointer, ldw, shuffled flag, dtype) of a row-major tensor or a ShuffledWeight."""
    if isinstance(weight, ShuffledWeight):
        return weight.n, weight.k, _dev(weight.data), weight.k_steps, 1, weight.dtype
    n, k, ldw = _rows(weight, "weight")
    return n, k, _dev(weight), ldw, 0, weight.dtype


def linear_workspace_bytes(dtype, max_rows, n, k):
    return int(library().tw_linear_workspace_bytes(dtype_id(dtype), int(max_rows), int(n), int(k)))


def linear_partial_splits(dtype, n, k):
    """K ranges `linear_partials` uses for an [n, k] weight; 0 if the shape is not supported."""
    return int(library().tw_linear_partial_splits(dtype_id(dtype), int(n), int(k)))


def linear_partial_splits_rows(weight, rows, lda=None):
    """K ranges `linear_partials` uses for ROWS rows (LDA elements apart, default: contiguous) against WEIGHT;
    0 where it cannot or would not split (above 64 rows the tiled kernels decide, and split only where whole
    tiles would leave CUs idle; which of them runs depends on the rows' stride too)."""
    n, k, _, _, shuffled, w_dtype = _weight_args(weight)
    return int(library().tw_linear_partial_splits_rows(dtype_id(w_dtype), shuffled, int(rows), n, k,
                                                       int(lda if lda is not None else k)))


def linear_partials(x, weight, partial):
    """partial[s] = x[:, K range s] @ weight[:, K range s].T in float32, for the K ranges
    `linear_partial_splits_rows` names for these rows.

    The caller's next kernel adds the splits up.
    """
    m, kx, lda = _rows(x, "x")
    n, k, w_ptr, ldw, shuffled, w_dtype = _weight_args(weight)
    _need(kx == k, "linear_partials shapes do not agree")
    _need(x.dtype == w_dtype and m >= 1, "linear_partials takes rows of the weight's type")
    splits = linear_partial_splits_rows(weight, m, lda)
    _need(splits > 0, "linear_partials: K must be a multiple of 16 bytes, and above 64 rows the shape must be one the tiled kernels split")
    _need(partial.is_contiguous() and tuple(partial.shape) == (splits, m, n), f"partial must be [{splits}, {m}, {n}]")
    check(library().tw_linear_partials(dtype_id(x.dtype), _dev(x), lda, w_ptr, ldw, shuffled,
                                       _dev(partial, torch.float32, "partial"), partial.numel() * 4, m, n, k,
                                       _stream()), "linear_partials")
    return partial


def interleave_glu_rows(gate, up):
    """[2n, k] with the rows of gate and up [n, k] alternating in blocks of 16 (n a multiple of 16).

    The same order applies to biases ([n] each). This is the row order `linear_glu` expects.
    """
    _need(gate.shape == up.shape and gate.shape[0] % 16 == 0, "gate and up must have equally many rows, a multiple of 16")
    n = gate.shape[0]
    rest = tuple(gate.shape[1:])
    return torch.stack([gate.reshape(n // 16, 16, *rest), up.reshape(n // 16, 16, *rest)], 1).reshape(2 * n, *rest).contiguous()


GLU_ACTIVATIONS = {"silu": 0, "gelu_tanh": 1, "swish_limited": 2}


def linear_glu(x, weight, out, bias=None, force=0, activation="silu", factor=1.0):
    """out[m, n/2] = factor * act(x @ gate.T) * (x @ up.T), weight [n, k] holding gate and up rows
    interleaved by `interleave_glu_rows` (row-major or shuffled); out has x's type. act is SiLU or the tanh
    form of gelu; the factor is applied in float32 before the rounding. With "swish_limited" the factor is a limit L
    instead: out = g' * sigmoid(1.702 g') * (u' + 1), g' = min(gate, L), u' = clamp(up, -L, L)."""
    _need(activation in GLU_ACTIVATIONS, f"activation must be one of {sorted(GLU_ACTIVATIONS)}")
    m, k, lda = _rows(x, "x")
    n, k2, w_ptr, ldw, shuffled, w_dtype = _weight_args(weight)
    mo, no, ldc = _rows(out, "out")
    _need(n % 32 == 0, "a gated weight has a multiple of 32 rows")
    _need(k == k2 and mo == m and no == n // 2, f"linear_glu shapes do not agree: x {tuple(x.shape)}, weight {(n, k2)}, out {tuple(out.shape)}")
    _need(x.dtype == w_dtype and out.dtype == x.dtype, "x, weight and out types differ")
    if bias is not None:
        _need(bias.numel() == n, "bias has the wrong size")
    check(library().tw_linear_glu(dtype_id(x.dtype), _dev(x), lda, w_ptr, ldw, shuffled,
                                  _dev(bias, torch.float32, "bias") if bias is not None else None,
                                  _dev(out), ldc, m, n, k, force, GLU_ACTIVATIONS[activation], float(factor), _stream()),
          "linear_glu")
    return out


GEMM_AUTO, GEMM_GENERIC, GEMM_TILED, GEMM_TILED_WIDE, GEMM_SKINNY, GEMM_TILED_256, GEMM_TILED_256X192, GEMM_STREAM_CU = 0, 1, 3, 4, 5, 6, 7, 8


def linear(x, weight, out, bias=None, residual=None, workspace=None, force=GEMM_AUTO):
    """out = x @ weight.T (+ bias) (+ residual).

    x [m, k] and weight [n, k] (a row-major tensor or a ShuffledWeight) share a type (float32 or
    bfloat16); out is float32 (required with a residual; the residual may be `out` itself) or that
    type. bias is float32 [n]; workspace is a float32/byte scratch tensor for split-K.
    """
    m, k, lda = _rows(x, "x")
    n, k2, w_ptr, ldw, shuffled, w_dtype = _weight_args(weight)
    mo, no, ldc = _rows(out, "out")
    _need(k == k2 and mo == m and no == n, f"linear shapes do not agree: x {tuple(x.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    _need(x.dtype == w_dtype, "x and weight types differ")
    out_f32 = out.dtype == torch.float32
    _need(out_f32 or out.dtype == x.dtype, "out must be float32 or the input type")
    ldr = 0
    if residual is not None:
        _need(out_f32, "a residual needs a float32 output")
        mr, nr, ldr = _rows(residual, "residual")
        _need((mr, nr) == (m, n), "residual shape differs from the output")
    if bias is not None:
        _need(bias.numel() == n and bias.is_contiguous(), "bias has the wrong size")
    ws_ptr, ws_bytes = None, 0
    if workspace is not None:
        ws_ptr, ws_bytes = _dev(workspace), workspace.numel() * workspace.element_size()
    check(library().tw_linear(dtype_id(x.dtype), 1 if out_f32 else 0, _dev(x), lda, w_ptr, ldw, shuffled,
                              _dev(bias, torch.float32, "bias") if bias is not None else None,
                              _dev(residual, torch.float32, "residual") if residual is not None else None, ldr,
                              _dev(out), ldc, ws_ptr, ws_bytes, m, n, k, int(force), _stream()), "linear")
    return out


LINEAR_ACTIVATIONS = {"relu_squared": 1, "gelu": 2}


def can_linear_act(x, weight):
    """Does `linear_act` take these operands? (more than 64 rows, K a multiple of 16 bytes: the tiled kernels)"""
    k = weight.shape[1]
    return x.shape[0] > 64 and k % (16 // x.element_size()) == 0


def linear_act(x, weight, out, activation="relu_squared", bias=None, workspace=None):
    """out = act(x @ weight.T + bias) in x's type, the activation applied in float32 in the matrix kernel's epilogue
    (or where its split-K sums are added up) before the one rounding. For more than 64 rows (`can_linear_act`)."""
    _need(activation in LINEAR_ACTIVATIONS, f"activation must be one of {sorted(LINEAR_ACTIVATIONS)}")
    m, k, lda = _rows(x, "x")
    n, k2, w_ptr, ldw, shuffled, w_dtype = _weight_args(weight)
    mo, no, ldc = _rows(out, "out")
    _need(k == k2 and mo == m and no == n, f"linear_act shapes do not agree: x {tuple(x.shape)}, weight {(n, k2)}, out {tuple(out.shape)}")
    _need(x.dtype == w_dtype == out.dtype and can_linear_act(x, weight), "linear_act takes more than 64 rows of the weight's type")
    if bias is not None:
        _need(bias.numel() == n and bias.is_contiguous(), "bias has the wrong size")
    ws_ptr, ws_bytes = None, 0
    if workspace is not None:
        ws_ptr, ws_bytes = _dev(workspace), workspace.numel() * workspace.element_size()
    check(library().tw_linear_act(dtype_id(x.dtype), _dev(x), lda, w_ptr, ldw, shuffled,
                                  _dev(bias, torch.float32, "bias") if bias is not None else None, _dev(out), ldc,
                                  ws_ptr, ws_bytes, m, n, k, LINEAR_ACTIVATIONS[activation], _stream()), "linear_act")
    return out


def attn_decode_splits(n_seqs, q_heads, kv_heads, max_kv_len):
    return int(library().tw_attn_decode_splits(n_seqs, q_heads, kv_heads, max_kv_len))


def attn_decode_workspace_floats(n_seqs, q_heads, head_dim, splits):
    return int(library().tw_attn_decode_workspace_floats(n_seqs, q_heads, head_dim, splits))


def _check_attention(q, keys, values, block_table, q_start, kv_len, out, q_heads, kv_heads, head_dim):
    nq, wq, ldq = _rows(q, "q")
    no, wo, ldo = _rows(out, "out")
    _need(wq >= q_heads * head_dim and wo == q_heads * head_dim and no == nq, "attention q/out shapes do not agree")
    _need(out.dtype == q.dtype == keys.dtype == values.dtype, "attention operand types differ")
    _need(keys.dim() == 4 and keys.is_contiguous() and values.is_contiguous() and values.numel() == keys.numel(),
          "keys must be contiguous [pages, kv_heads, page_size, head_dim] and values the same size")
    _need(keys.shape[1] == kv_heads and keys.shape[3] == head_dim, "cache shape does not match the head sizes")
    _need(head_dim % 16 == 0 and 16 <= head_dim <= 256, "head_dim must be a multiple of 16 between 16 and 256")
    _need(keys.shape[2] % 4 == 0, "page_size must be a multiple of 4")
    _need(q_heads % kv_heads == 0, "q_heads must be a multiple of kv_heads")
    _need(block_table.dim() == 2 and block_table.stride(1) == 1, "block_table must be 2-D")
    _need(q_start.numel() >= kv_len.numel() + 1, "q_start needs one more entry than kv_len")
    return ldq, ldo


def attn_decode(q, keys, values, block_table, q_start, kv_len, seq0, n_seqs, out, q_heads, kv_heads,
                head_dim, scale, window=0, splits=1, workspace=None, generic=False, softcap=0.0):
    """Attention of sequences seq0..seq0+n_seqs-1, each with ONE query token, over their pages.

    generic=True forces the kernel that takes every type and page size (bfloat16 with
    pages of a multiple of 8 keys otherwise runs a faster kernel of its own). softcap > 0 passes the scaled
    scores through softcap * tanh(score / softcap).
    """
    ldq, ldo = _check_attention(q, keys, values, block_table, q_start, kv_len, out, q_heads, kv_heads, head_dim)
    _need(seq0 + n_seqs <= kv_len.numel() and seq0 + n_seqs <= block_table.shape[0], "sequence range exceeds the metadata")
    ws_ptr, ws_floats = None, 0
    if splits > 1:
        _need(workspace is not None and workspace.dtype == torch.float32, "split decode attention needs a float32 workspace")
        ws_ptr, ws_floats = _dev(workspace), workspace.numel()
    check(library().tw_attn_decode(dtype_id(q.dtype), _dev(q), ldq, _dev(keys), _dev(values),
                                   _dev(block_table, torch.int32, "block_table"), block_table.stride(0),
                                   _dev(q_start, torch.int32, "q_start"), _dev(kv_len, torch.int32, "kv_len"),
                                   seq0, n_seqs, _dev(out), ldo, ws_ptr, ws_floats, q_heads, kv_heads, head_dim,
                                   keys.shape[2], int(window or 0), float(scale), float(softcap or 0.0), int(splits),
                                   1 if generic else 0, _stream()),
          "attn_decode")
    return out


def attn_prefill_split(n_seqs, q_heads, kv_heads, max_q_len, max_kv_len, tile_rows=0):
    """(max_chunks, kv_chunk, tile_rows): how the fast prefill kernel would cut the keys of a tile into
    chunks that separate workgroups take (max_chunks == 1: not at all) for a launch of this shape, and the
    rows of a workgroup's tile it would use (tile_rows 64 or 128 asks for that size)."""
    import ctypes
    chunk, rows = ctypes.c_int(0), ctypes.c_int(0)
    chunks = int(library().tw_attn_prefill_split(int(n_seqs), q_heads, kv_heads, int(max_q_len), int(max_kv_len),
                                                 int(tile_rows), ctypes.byref(chunk), ctypes.byref(rows)))
    return chunks, int(chunk.value), int(rows.value)


def attn_prefill_workspace_floats(n_tokens, q_heads, head_dim, max_chunks):
    return int(library().tw_attn_prefill_workspace_floats(int(n_tokens), q_heads, head_dim, int(max_chunks)))


def attn_prefill(q, keys, values, block_table, q_start, kv_len, seq0, n_seqs, max_q_len, out, q_heads,
                 kv_heads, head_dim, scale, window=0, generic=False, split=None, workspace=None, softcap=0.0, sink=None,
                 stats=None):
    """Attention of sequences seq0..seq0+n_seqs-1 with up to max_q_len query tokens each.

    sink float32 [q_heads]: exp(sink_h) more in head h's softmax denominator (a score of its own, not scaled, with
    no key and no value). stats float32 [rows of q, q_heads, 2]: gets what each row's softmax was taken against (a scaled
    score) and the row's sum relative to it, for `attn_kept_keys`.

    split = (max_chunks, kv_chunk[, tile_rows]) from attn_prefill_split with a float32 workspace of
    attn_prefill_workspace_floats(rows of q, ...) lets the fast bfloat16 kernel cut long key ranges
    into chunks for separate workgroups (a second kernel merges them in a fixed order).
    """
    ldq, ldo = _check_attention(q, keys, values, block_table, q_start, kv_len, out, q_heads, kv_heads, head_dim)
    _need(seq0 + n_seqs <= kv_len.numel() and seq0 + n_seqs <= block_table.shape[0], "sequence range exceeds the metadata")
    _need(sink is None or (sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == q_heads), "sink must be float32 [q_heads]")
    _need(stats is None or (stats.dtype == torch.float32 and stats.is_contiguous() and stats.numel() >= q.shape[0] * q_heads * 2),
          "stats must be float32 [rows, q_heads, 2]")
    max_chunks, kv_chunk, ws_ptr, ws_floats = 1, 0, None, 0
    tile_rows = int(split[2]) if split is not None and len(split) > 2 else 0
    if split is not None and split[0] > 1:
        max_chunks, kv_chunk = int(split[0]), int(split[1])
        _need(workspace is not None and workspace.dtype == torch.float32, "split prefill attention needs a float32 workspace")
        ws_ptr, ws_floats = _dev(workspace), workspace.numel()
    check(library().tw_attn_prefill(dtype_id(q.dtype), _dev(q), ldq, _dev(keys), _dev(values),
                                    _dev(block_table, torch.int32, "block_table"), block_table.stride(0),
                                    _dev(q_start, torch.int32, "q_start"), _dev(kv_len, torch.int32, "kv_len"),
                                    seq0, n_seqs, int(max_q_len), _dev(out), ldo, ws_ptr, ws_floats, q.shape[0],
                                    max_chunks, kv_chunk, tile_rows, q_heads, kv_heads, head_dim,
                                    keys.shape[2], int(window or 0), float(scale), float(softcap or 0.0),
                                    1 if generic else 0, _dev(sink) if sink is not None else None,
                                    _dev(stats) if stats is not None else None, _stream()), "attn_prefill")
    return out


def attn_kept_keys(q, keys, values, block_table, q_start, kv_len, seq0, n_seqs, row0, n_rows, out, stats, q_heads, kv_heads,
                   head_dim, scale, window, keep_first, sink=None):
    """Completes rows row0 .. row0 + n_rows - 1 (those of sequences seq0 .. seq0 + n_seqs - 1, in order) of a windowed
    `attn_prefill` that left `stats`: adds the sequence's first keep_first keys as far as they lie before a row's window,
    and the sink, and writes out anew. Same cache layout as `attn_prefill`."""
    ldq, ldo = _check_attention(q, keys, values, block_table, q_start, kv_len, out, q_heads, kv_heads, head_dim)
    _need(stats.dtype == torch.float32 and stats.is_contiguous() and stats.numel() >= q.shape[0] * q_heads * 2,
          "stats must be float32 [rows, q_heads, 2]")
    _need(row0 + n_rows <= q.shape[0] and seq0 + n_seqs <= kv_len.numel() and seq0 + n_seqs <= block_table.shape[0],
          "rows or sequences exceed the step")
    _need(sink is None or (sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == q_heads), "sink must be float32 [q_heads]")
    check(library().tw_attn_kept_keys(dtype_id(q.dtype), _dev(q), ldq, _dev(keys), _dev(values),
                                      _dev(block_table, torch.int32, "block_table"), block_table.stride(0),
                                      _dev(q_start, torch.int32, "q_start"), _dev(kv_len, torch.int32, "kv_len"), int(seq0),
                                      int(n_seqs), int(row0), int(n_rows), _dev(out), ldo, _dev(stats),
                                      _dev(sink) if sink is not None else None, q_heads, kv_heads, head_dim, keys.shape[2],
                                      int(window or 0), int(keep_first or 0), float(scale), _stream()), "attn_kept_keys")
    return out


def sampling_uniform(seed, counter):
    """The uniform number the sampler draws for (seed, counter); host-side, for tests."""
    return float(library().tw_sampling_uniform(int(seed) & (2 ** 64 - 1), int(counter)))


def sample_workspace_bytes(rows):
    return int(library().tw_sample_workspace_bytes(int(rows)))


def sample_rows(logits, out, temperature=None, seeds=None, counters=None, workspace=None):
    """out[r] = greedy (temperature 0 or None) or sampled token of logits[r].

    workspace: a device tensor of at least sample_workspace_bytes(rows) bytes (allocated here if None).
    """
    rows, vocab, ld = _rows(logits, "logits")
    _need(out.numel() == rows, "one output id per row is needed")
    need = sample_workspace_bytes(rows)
    if workspace is None:
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=logits.device)
    _need(workspace.is_contiguous() and workspace.numel() * workspace.element_size() >= need,
          "the sampling workspace is too small")
    if temperature is not None:
        _need(temperature.numel() == rows and seeds.numel() == rows and counters.numel() == rows,
              "one temperature, seed and counter per row are needed")
        _need(seeds.dtype == torch.int64, "seeds must be int64")
    check(library().tw_sample_rows(_dev(logits, torch.float32, "logits"), ld, rows, vocab,
                                   _dev(temperature, torch.float32, "temperature") if temperature is not None else None,
                                   _dev(seeds) if temperature is not None else None,
                                   _dev(counters, torch.int32, "counters") if temperature is not None else None,
                                   _dev(out, torch.int32, "out"), _dev(workspace),
                                   workspace.numel() * workspace.element_size(), _stream()), "sample_rows")
    return out


# ---- kernels over sequences: position table, causal convolution with state, gated recurrence, layer end ---------

def add_table_rows(x, table, ids, copy=None):
    """x[n] += table[ids[n]] (x float32 [n, width]); COPY, if given, receives the sums as well."""
    n, width = x.shape
    _need(x.is_contiguous() and table.dim() == 2 and table.is_contiguous() and table.shape[1] == width,
          "add_table_rows: x [n, width] and table [rows, width] must be contiguous")
    _need(ids.numel() == n, "one row id per token is needed")
    if copy is not None:
        _need(copy.is_contiguous() and tuple(copy.shape) == (n, width), "the copy must have x's shape")
    check(library().tw_add_table_rows(dtype_id(table.dtype), _dev(x, torch.float32, "x"), _dev(table),
                                      _dev(ids, torch.int32, "ids"), n, width, table.shape[0],
                                      _dev(copy, torch.float32, "copy") if copy is not None else None, _stream()),
          "add_table_rows")
    return x


CONV_MAX_TAPS = 8


CONV_ACTIVATIONS = {None: 0, "silu": 1}


def causal_conv(src, taps, state, q_start, kv_len, state_slots, phase, n_seqs, out=None, out32=None, norm_weight=None,
                eps=0.0, bias=None, identity=0.0, row_scratch=None, activation=None):
    """Causal convolution over time on each channel, with the request's last inputs as state.

    v_t = src_t (or its RMS norm times norm_weight, for float32 rows); out_t = identity * v_t +
    sum_j taps[:, j] * v_(t - K + 1 + j) + bias. state float32 [requests, 2, max(K - 1, 1), C]: copy
    phase[s] is read, the other copy written. out has the compute type, out32 is float32; either may be None.
    row_scratch: float32 [>= n]; with a norm and many rows the rows' statistics are then formed once by a kernel of
    their own. activation "silu": out_t passes SiLU before it is written (the state keeps the inputs v, as always).
    """
    _need(activation in CONV_ACTIVATIONS, "a convolution's activation is None or 'silu'")
    n, C, ld_src = _rows(src, "src")
    K = taps.shape[1]
    _need(taps.dtype == torch.float32 and taps.is_contiguous() and taps.shape[0] == C, "taps must be float32 [C, K]")
    _need(1 <= K <= CONV_MAX_TAPS, f"a convolution has 1 to {CONV_MAX_TAPS} taps")
    _need(state.dtype == torch.float32 and state.is_contiguous() and state.dim() == 4
          and tuple(state.shape[1:]) == (2, max(K - 1, 1), C), "state must be float32 [requests, 2, max(K - 1, 1), C]")
    _need(out is not None or out32 is not None, "causal_conv needs an output")
    ld_out = ld_out32 = 0
    compute = src.dtype
    if out is not None:
        no, co, ld_out = _rows(out, "out")
        _need((no, co) == (n, C), "out has the wrong shape")
        compute = out.dtype
    if out32 is not None:
        no, co, ld_out32 = _rows(out32, "out32")
        _need((no, co) == (n, C) and out32.dtype == torch.float32, "out32 must be float32 [n, C]")
    src_f32 = src.dtype == torch.float32
    _need(src_f32 or src.dtype == compute, "src must be float32 or of the output's type")
    if norm_weight is not None:
        _need(src_f32 and norm_weight.numel() == C, "a norm needs float32 rows and a weight per channel")
    if bias is not None:
        _need(bias.numel() == C and bias.dtype == torch.float32, "bias must be float32 [C]")
    _need(q_start.numel() >= n_seqs + 1 and kv_len.numel() >= n_seqs and state_slots.numel() >= n_seqs
          and phase.numel() >= n_seqs, "sequence metadata is too short")
    use_scratch = row_scratch is not None and norm_weight is not None
    if use_scratch:
        _need(row_scratch.is_contiguous() and row_scratch.numel() >= n, "row_scratch must hold a float per row")
    check(library().tw_causal_conv(dtype_id(compute), 1 if src_f32 else 0, _dev(src), ld_src,
                                   _dev(norm_weight, torch.float32, "norm_weight") if norm_weight is not None else None,
                                   float(eps), _dev(taps), _dev(bias) if bias is not None else None, float(identity),
                                   _dev(state), _dev(q_start, torch.int32, "q_start"), _dev(kv_len, torch.int32, "kv_len"),
                                   _dev(state_slots, torch.int32, "state_slots"), _dev(phase, torch.int32, "phase"),
                                   _dev(out) if out is not None else None, ld_out,
                                   _dev(out32) if out32 is not None else None, ld_out32, n, int(n_seqs), C, K,
                                   _dev(row_scratch, torch.float32, "row_scratch") if use_scratch else None,
                                   CONV_ACTIVATIONS[activation], _stream()),
          "causal_conv")


def gated_recurrence_workspace_floats(n_seqs, max_q_len, channels):
    return int(library().tw_gated_recurrence_workspace_floats(int(n_seqs), int(max_q_len), int(channels)))


def gated_recurrence(gates, u, branch, lam, state, q_start, state_slots, n_seqs, max_q_len, out, blocks, decay,
                     out_scale=1.0, out_pad=0, workspace=None):
    """The gated linear recurrence S = a S + sqrt(1 - a^2) i u per sequence and channel, a = exp(-decay *
    sigmoid(gate_a) * softplus(lam)); out = out_scale * S * gelu_tanh(branch). gates float32 [n, 2C], block b's
    recurrence gates at columns [2 b C/blocks, ...) followed by its input gates; u float32 [n, C]; branch and
    out have the compute type; state float32 [requests, C]. max_q_len: the longest portion of the step; portions
    longer than a chunk are walked by several threads a channel and need a float32 workspace
    (`gated_recurrence_workspace_floats`). out_pad: further columns of out that are set to zero."""
    n, C, ld_u = _rows(u, "u")
    ng, cg, ld_g = _rows(gates, "gates")
    nb, cb, ld_b = _rows(branch, "branch")
    no, co, ld_o = _rows(out, "out")
    _need(gates.dtype == torch.float32 and u.dtype == torch.float32, "gates and u must be float32")
    _need((ng, cg) == (n, 2 * C) and (nb, cb) == (n, C) and (no, co) == (n, C + out_pad) and branch.dtype == out.dtype,
          "gated_recurrence shapes do not agree")
    _need(C % blocks == 0 and lam.numel() == C and lam.dtype == torch.float32, "lam must be float32 [C], C a multiple of blocks")
    _need(state.dtype == torch.float32 and state.is_contiguous() and state.shape[-1] == C and state.dim() == 2,
          "state must be float32 [requests, C]")
    _need(q_start.numel() >= n_seqs + 1 and state_slots.numel() >= n_seqs and 1 <= max_q_len, "sequence metadata is too short")
    need = gated_recurrence_workspace_floats(n_seqs, max_q_len, C)
    if need:
        _need(workspace is not None and workspace.dtype == torch.float32 and workspace.numel() >= need,
              "portions longer than a chunk need a float32 workspace")
    check(library().tw_gated_recurrence(dtype_id(out.dtype), _dev(gates), ld_g, _dev(u), ld_u, _dev(branch), ld_b,
                                        _dev(lam), _dev(state), _dev(q_start, torch.int32, "q_start"),
                                        _dev(state_slots, torch.int32, "state_slots"), _dev(out), ld_o, int(n_seqs),
                                        int(max_q_len), C, int(blocks), int(out_pad), float(decay), float(out_scale),
                                        _dev(workspace) if need else None, workspace.numel() if need else 0, _stream()),
          "gated_recurrence")
    return out


def can_block_diagonal(x, weight):
    """Does `block_diagonal` take these operands? (blocks of a multiple of 16 bytes in, a multiple of 16 out, aligned rows)"""
    epf = 16 // x.element_size()
    blocks, n_out, n_in = weight.shape
    return (n_in % epf == 0 and n_out % 16 == 0 and x.stride(0) % epf == 0 and x.data_ptr() % 16 == 0
            and x.shape[1] == blocks * n_in)


def block_diagonal(x, weight, bias, out):
    """out[n, b * No + o] = sum_i x[n, b * Ni + i] * weight[b, o, i] + bias[b * No + o]; weight [blocks, No, Ni] of x's
    type, out float32 [n, blocks * No]."""
    n, width, ldx = _rows(x, "x")
    blocks, n_out, n_in = weight.shape
    no, wo, ldo = _rows(out, "out")
    _need(weight.is_contiguous() and weight.dtype == x.dtype and can_block_diagonal(x, weight), "block_diagonal: unsupported operands")
    _need(out.dtype == torch.float32 and (no, wo) == (n, blocks * n_out) and ldo % 4 == 0 and out.data_ptr() % 16 == 0,
          "out must be float32 [n, blocks * No] with 16-byte aligned rows")
    _need(bias is None or (bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == blocks * n_out), "bias has the wrong size")
    check(library().tw_block_diagonal(dtype_id(x.dtype), _dev(x), ldx, _dev(weight), _dev(bias) if bias is not None else None,
                                      _dev(out), ldo, n, blocks, n_in, n_out, _stream()), "block_diagonal")
    return out


def gelu_mul(gate_up, out, scale=1.0):
    """out[n, i] = scale * gelu_tanh(gate_up[n, i]) * gate_up[n, inter + i]."""
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 2 == 0, "gate_up must be contiguous [n, 2*inter]")
    n, inter = gate_up.shape[0], gate_up.shape[1] // 2
    _need(out.is_contiguous() and tuple(out.shape) == (n, inter) and out.dtype == gate_up.dtype,
          "gelu_mul output has the wrong shape or type")
    check(library().tw_gelu_mul(dtype_id(gate_up.dtype), _dev(gate_up), _dev(out), n, inter, float(scale), _stream()), "gelu_mul")
    return out


def round_rows(x, out):
    """out = x rounded to out's type (x float32, both contiguous and of one shape)."""
    _need(x.is_contiguous() and out.is_contiguous() and x.shape == out.shape, "round_rows operands must be contiguous and alike")
    check(library().tw_round_rows(dtype_id(out.dtype), _dev(x, torch.float32, "x"), _dev(out), x.numel(), _stream()), "round_rows")
    return out


def token_gate(pre, table, ids, offset, out, feed=None):
    """out[n, k] = gelu_tanh(pre[n, k]) * table[ids[n], offset + k]; an id -1 - k stands for feed[k]."""
    n, dim = pre.shape
    _need(pre.dtype == torch.float32 and pre.is_contiguous() and out.is_contiguous() and tuple(out.shape) == (n, dim),
          "token_gate: pre float32 [n, dim] and out [n, dim] must be contiguous")
    _need(table.dim() == 2 and table.is_contiguous() and table.dtype == out.dtype and offset + dim <= table.shape[1],
          "token_gate: the table must be contiguous, of out's type, and hold the asked columns")
    check(library().tw_token_gate(dtype_id(out.dtype), _dev(pre), _dev(table), table.shape[1], _dev(ids, torch.int32, "ids"),
                                  _dev(feed, torch.int32, "feed") if feed is not None else None,
                                  feed.numel() if feed is not None else 0, table.shape[0], int(offset), _dev(out), n, dim,
                                  _stream()), "token_gate")
    return out


def layer_end(x, layer, branch=None, branch_weight=None, eps=0.0, mult=1.0, history=None, mix=None):
    """x += mult * branch / rms(branch) * branch_weight (if a branch is given); history[layer + 1] = x;
    then, with MIX (float32 [layer + 2]), x = sum_j mix[j] * history[j]. history float32 [layers + 1, rows, width]
    (rows >= n: a buffer sized for the largest step)."""
    n, width = x.shape
    _need(x.dtype == torch.float32 and x.is_contiguous(), "x must be contiguous float32 [n, width]")
    if branch is not None:
        _need(branch.dtype == torch.float32 and branch.is_contiguous() and tuple(branch.shape) == (n, width)
              and branch_weight is not None and branch_weight.numel() == width, "the branch must be float32 [n, width] with a weight")
    stride = 0
    if history is not None:
        _need(history.dtype == torch.float32 and history.is_contiguous() and history.dim() == 3
              and history.shape[2] == width and history.shape[1] >= n and history.shape[0] >= layer + 2,
              "history must be float32 [layers + 1, rows >= n, width]")
        stride = history.shape[1] * width
    if mix is not None:
        _need(history is not None and mix.dtype == torch.float32 and mix.numel() == layer + 2, "mix must be float32 [layer + 2]")
    check(library().tw_layer_end(_dev(x), _dev(branch) if branch is not None else None,
                                 _dev(branch_weight, torch.float32, "branch_weight") if branch is not None else None,
                                 float(eps), float(mult), _dev(history) if history is not None else None, stride, int(layer),
                                 _dev(mix) if mix is not None else None, n, width, _stream()), "layer_end")
    return x


# ---- attention with scores mixed across heads ------------------------------------------------------------------------

def attn_mixed_splits(n_seqs, max_kv_len):
    return int(library().tw_attn_mixed_splits(int(n_seqs), int(max_kv_len)))


def attn_mixed_prefill_splits(n_tokens, n_seqs, max_kv_len):
    """Key ranges for a launch over prompt portions (1: none): more than one only where there are few row tiles."""
    return int(library().tw_attn_mixed_prefill_splits(int(n_tokens), int(n_seqs), int(max_kv_len)))


def attn_mixed_workspace_floats(n_seqs, max_q_len, q_heads, value_dim, splits):
    return int(library().tw_attn_mixed_workspace_floats(int(n_seqs), int(max_q_len), q_heads, value_dim, int(splits)))


def kv_store(src, k_col, v_col, slots, keys, values, kv_heads, key_dim, value_dim):
    """Row n's keys src[n, k_col : k_col + kv_heads * key_dim] and values src[n, v_col : ...] into the page slot
    slots[n] (-1: not stored). keys [pages, kv_heads, page, key_dim]; values [pages, kv_heads, value_dim, page]."""
    n, width, ld = _rows(src, "src")
    page = keys.shape[2]
    _need(keys.is_contiguous() and values.is_contiguous() and keys.dtype == src.dtype == values.dtype, "cache and source types differ")
    _need(tuple(keys.shape[1:]) == (kv_heads, page, key_dim) and tuple(values.shape[1:]) == (kv_heads, value_dim, page)
          and values.shape[0] == keys.shape[0], "keys [pages, kv_heads, page, key_dim], values [pages, kv_heads, value_dim, page]")
    _need(k_col + kv_heads * key_dim <= width and v_col + kv_heads * value_dim <= width and slots.numel() == n,
          "kv_store: columns exceed the rows, or not one slot per row")
    check(library().tw_kv_store(dtype_id(src.dtype), _dev(src), ld, int(k_col), int(v_col), _dev(slots, torch.int32, "slots"),
                                _dev(keys), _dev(values), n, kv_heads, key_dim, value_dim, page, _stream()), "kv_store")


def attn_mixed(q, keys, values, block_table, q_start, kv_len, seq0, n_seqs, max_q_len, out, q_heads, kv_heads, scale,
               window=0, talk=None, sink=None, slopes=None, out_scale=1.0, splits=1, workspace=None, keep_first=0):
    """Attention of sequences seq0 .. seq0 + n_seqs - 1 whose scores are mixed across heads before the softmax.

    q [rows, >= q_heads * key_dim] (head h at columns h * key_dim), keys [pages, kv_heads, page, key_dim], values
    [pages, kv_heads, value_dim, page], out [rows, q_heads * value_dim]. talk float32 [H, H] mixes the scores
    (None: no mixing), slopes float32 [H] take slope * distance off the raw scores, sink float32 [H] adds exp(sink)
    to the softmax's denominator. keep_first: with a window, the sequence's first keep_first keys stay visible to every later
    query (at their true positions). splits > 1 cuts every tile's keys into ranges; needs a workspace
    (`attn_mixed_workspace_floats`).
    """
    key_dim, value_dim, page = keys.shape[3], values.shape[2], keys.shape[2]
    nq, wq, ldq = _rows(q, "q")
    no, wo, ldo = _rows(out, "out")
    _need(wq >= q_heads * key_dim and wo == q_heads * value_dim and no == nq, "attention q/out shapes do not agree")
    _need(out.dtype == q.dtype == keys.dtype == values.dtype, "attention operand types differ")
    _need(keys.dim() == 4 and values.dim() == 4 and keys.is_contiguous() and values.is_contiguous()
          and keys.shape[1] == kv_heads and tuple(values.shape[:2]) == tuple(keys.shape[:2]) and values.shape[3] == page,
          "keys [pages, kv_heads, page, key_dim] and values [pages, kv_heads, value_dim, page] are needed")
    _need(block_table.dim() == 2 and block_table.stride(1) == 1, "block_table must be 2-D")
    _need(seq0 + n_seqs <= kv_len.numel() and seq0 + n_seqs <= block_table.shape[0] and q_start.numel() >= seq0 + n_seqs + 1,
          "sequence range exceeds the metadata")
    for name, t, count in (("talk", talk, q_heads * q_heads), ("sink", sink, q_heads), ("slopes", slopes, q_heads)):
        _need(t is None or (t.dtype == torch.float32 and t.is_contiguous() and t.numel() == count), f"{name} has the wrong size or type")
    ws_ptr, ws_floats = None, 0
    if splits > 1:
        _need(workspace is not None and workspace.dtype == torch.float32, "split attention needs a float32 workspace")
        ws_ptr, ws_floats = _dev(workspace), workspace.numel()
    check(library().tw_attn_mixed(dtype_id(q.dtype), _dev(q), ldq, _dev(keys), _dev(values),
                                  _dev(block_table, torch.int32, "block_table"), block_table.stride(0),
                                  _dev(q_start, torch.int32, "q_start"), _dev(kv_len, torch.int32, "kv_len"), int(seq0),
                                  int(n_seqs), int(max_q_len), _dev(out), ldo,
                                  _dev(talk) if talk is not None else None, _dev(sink) if sink is not None else None,
                                  _dev(slopes) if slopes is not None else None, ws_ptr, ws_floats, q_heads, kv_heads,
                                  key_dim, value_dim, page, int(window or 0), int(keep_first or 0), float(scale), float(out_scale), int(splits),
                                  _stream()), "attn_mixed")
    return out


# ---- norm after the sum, relu squared, hashed pair embedding ----------------------------------------------------------

def residual_norm(x, weight, eps, out=None, y=None, add=None, scale=None, alpha=1.0):
    """x <- weight * unit(alpha * x + scale * y), unit(v) = v / sqrt(mean(v^2) + eps); x float32 [n, hidden] in place.

    y: float32 [n, hidden] (rows may be strided), or add: float32 [splits, n, hidden] partial sums added up here;
    scale: float32 [hidden] or None; out: the normed rows once more, rounded to its type (the compute type)."""
    _need(x.dim() == 2 and x.is_contiguous() and x.dtype == torch.float32, "residual_norm: x must be contiguous float32 [n, hidden]")
    n, hidden = x.shape
    _need(weight.numel() == hidden and weight.dtype == torch.float32 and weight.is_contiguous(), "the norm weight must be float32 [hidden]")
    ldy = 0
    if y is not None:
        ny, cy, ldy = _rows(y, "y")
        _need((ny, cy) == (n, hidden) and y.dtype == torch.float32, "y must be float32 [n, hidden]")
    splits, stride = 0, 0
    if add is not None:
        _need(y is None, "either y or partial sums")
        _need(add.dim() == 3 and add.is_contiguous() and tuple(add.shape[1:]) == (n, hidden) and add.dtype == torch.float32,
              "partial sums must be float32 [splits, n, hidden]")
        splits, stride = add.shape[0], n * hidden
    if scale is not None:
        _need(scale.numel() == hidden and scale.dtype == torch.float32 and scale.is_contiguous(), "scale must be float32 [hidden]")
    out_dtype = F32
    if out is not None:
        _need(out.is_contiguous() and tuple(out.shape) == (n, hidden), "out must be contiguous [n, hidden]")
        out_dtype = dtype_id(out.dtype)
    check(library().tw_residual_norm(out_dtype, _dev(x), _dev(y) if y is not None else None, ldy,
                                     _dev(add) if add is not None else None, splits, stride,
                                     _dev(scale) if scale is not None else None, _dev(weight),
                                     _dev(out) if out is not None else None, n, hidden, float(alpha), float(eps), _stream()),
          "residual_norm")
    return x


def relu_squared(x, partial=None):
    """x <- max(x, 0)^2 in place (rows may be strided); with PARTIAL (float32 [splits, n, cols], split-K sums of the
    product before) x <- max(sum of the splits, 0)^2 instead, rounded once."""
    n, cols, ld = _rows(x, "x")
    splits = 0
    if partial is not None:
        _need(partial.dim() == 3 and partial.is_contiguous() and tuple(partial.shape[1:]) == (n, cols)
              and partial.dtype == torch.float32, "partial sums must be float32 [splits, n, cols]")
        splits = partial.shape[0]
    check(library().tw_relu_squared(dtype_id(x.dtype), _dev(x), ld, n, cols, _dev(partial) if partial is not None else None,
                                    splits, _stream()), "relu_squared")
    return x


def embed_hashed(ids, table, pairs, norm_weight, q_start, kv_len, state_slots, phase, state, n_seqs, buckets, mul_prev,
                 mul_cur, scale, eps, x, out=None, feed=None):
    """x[n] = norm_weight * unit(scale * table[ids[n]] + pairs[r]), r = (previous token * mul_prev + token * mul_cur) mod
    buckets, r = buckets for a sequence's first token. state int32 [requests, 2] holds the last token of every request
    twice (copy phase[s] is read, the other written). x float32 [n, hidden]; out: the same rounded to its type."""
    n = ids.numel()
    vocab, hidden = table.shape
    _need(table.is_contiguous() and pairs.is_contiguous() and pairs.dtype == table.dtype and tuple(pairs.shape) == (buckets + 1, hidden),
          "the pair table must be [buckets + 1, hidden] of the embedding's type")
    _need(x.is_contiguous() and tuple(x.shape) == (n, hidden) and x.dtype == torch.float32, "x must be float32 [n, hidden]")
    _need(norm_weight.numel() == hidden and norm_weight.dtype == torch.float32, "the norm weight must be float32 [hidden]")
    _need(state.dtype == torch.int32 and state.is_contiguous() and state.dim() == 2 and state.shape[1] == 2, "state must be int32 [requests, 2]")
    _need(q_start.numel() >= n_seqs + 1 and kv_len.numel() >= n_seqs and state_slots.numel() >= n_seqs and phase.numel() >= n_seqs,
          "sequence metadata is too short")
    if out is not None:
        _need(out.is_contiguous() and tuple(out.shape) == (n, hidden) and out.dtype == table.dtype, "out must be [n, hidden] of the table's type")
    check(library().tw_embed_hashed(dtype_id(table.dtype), _dev(ids, torch.int32, "ids"),
                                    _dev(feed, torch.int32, "feed") if feed is not None else None,
                                    feed.numel() if feed is not None else 0, _dev(table), _dev(pairs), _dev(norm_weight),
                                    _dev(q_start, torch.int32, "q_start"), _dev(kv_len, torch.int32, "kv_len"),
                                    _dev(state_slots, torch.int32, "state_slots"), _dev(phase, torch.int32, "phase"),
                                    _dev(state), n, int(n_seqs), hidden, vocab, int(buckets), int(mul_prev), int(mul_cur),
                                    float(scale), float(eps), _dev(x), _dev(out) if out is not None else None, _stream()),
          "embed_hashed")
    return x


# ---- attention over a cached latent: finishing a token's projections, one small matrix per head -----------------------

def latent_finish(proj, q_col, c_col, kr_col, cos, sin, norm_weight, q_out, heads, latent, latent_dev, rot_dev, eps,
                  keys=None, values=None, slots=None, q_full=None, dim=0, dim_dev=0, full_from=0):
    """Rotates the heads' rotated query parts proj[n, q_col + a * rot_dev ...] into q_out[n, a, latent_dev:], and,
    with keys/values, stores the token's key row [unit(proj[n, c_col : c_col + latent]) * norm_weight | zeros |
    rotated proj[n, kr_col ...] | zeros] and its value (the normed latent) into page slot slots[n] (-1: not stored).
    keys [pages, 1, page, latent_dev + rot_dev]; values [pages, 1, latent_dev, page]; q_out [n, heads * (latent_dev + rot_dev)].
    q_full [n, heads * hd]: rows from full_from on also get whole query heads [the head's dim unrotated elements (which lie
    first in proj, dim_dev apart) | its rotated part | zeros], for attention against keys expanded per head."""
    n, width, ld = _rows(proj, "proj")
    rot = 2 * cos.shape[1]
    _need(tuple(cos.shape) == (n, rot // 2) and tuple(sin.shape) == (n, rot // 2) and cos.is_contiguous() and sin.is_contiguous()
          and cos.dtype == torch.float32, "rotary tables must be float32 [n, rot / 2]")
    nq, wq, ldq = _rows(q_out, "q_out")
    K = latent_dev + rot_dev
    _need(nq == n and wq == heads * K and q_out.dtype == proj.dtype, "q_out must be [n, heads * (latent_dev + rot_dev)] of proj's type")
    _need(q_col + heads * rot_dev <= width and rot <= rot_dev, "the rotated query parts exceed the projection's row")
    page = 0
    if keys is not None:
        page = keys.shape[2]
        _need(keys.is_contiguous() and values.is_contiguous() and keys.dtype == proj.dtype == values.dtype, "cache and projection types differ")
        _need(tuple(keys.shape[1:]) == (1, page, K) and tuple(values.shape) == (keys.shape[0], 1, latent_dev, page),
              "keys [pages, 1, page, latent_dev + rot_dev], values [pages, 1, latent_dev, page]")
        _need(slots.numel() == n and norm_weight.numel() == latent and norm_weight.dtype == torch.float32 and latent <= latent_dev,
              "one slot per token and a float32 norm weight per latent element are needed")
        _need(c_col + latent <= width and kr_col + rot <= width, "the latent or the shared key part exceed the projection's row")
    ld_full = hd = 0
    if q_full is not None:
        nf, wf, ld_full = _rows(q_full, "q_full")
        hd = wf // heads
        _need(nf == n and wf == heads * hd and q_full.dtype == proj.dtype and hd >= dim + rot and dim_dev >= dim > 0
              and q_col >= heads * dim_dev, "q_full must be [n, heads * hd] with hd >= dim + rot")
    check(library().tw_latent_finish(dtype_id(proj.dtype), _dev(proj), ld, int(q_col), int(c_col), int(kr_col), _dev(cos), _dev(sin),
                                     _dev(norm_weight) if keys is not None else None, _dev(q_out), ldq,
                                     _dev(q_full) if q_full is not None else None, ld_full, int(dim), int(dim_dev), int(hd),
                                     int(full_from), _dev(keys) if keys is not None else None, _dev(values) if keys is not None else None,
                                     _dev(slots, torch.int32, "slots") if keys is not None else None, n, heads, int(latent),
                                     int(latent_dev), int(rot_dev), rot, page, float(eps), _stream()), "latent_finish")


def latent_decode_splits(n_seqs, heads, max_kv_len):
    return int(library().tw_latent_decode_splits(int(n_seqs), int(heads), int(max_kv_len)))


def latent_decode_workspace_floats(n_seqs, heads, latent_dev, splits):
    return int(library().tw_latent_decode_workspace_floats(int(n_seqs), int(heads), int(latent_dev), int(splits)))


def latent_decode(q, keys, values, block_table, q_start, kv_len, n_seqs, out, heads, scale, splits=1, workspace=None, sink=None):
    """Attention of sequences 0 .. n_seqs - 1, ONE query token each, all heads against the one cached head: softmax of
    scale * q_a . key over the sequence's keys, times the values (the first latent_dev elements of the key rows).
    q [rows, heads * K] (head a at a * K), keys [pages, 1, page, K], values [pages, 1, latent_dev, page] (the same
    elements, transposed inside a page), out [rows, heads * latent_dev]. splits > 1 cuts every sequence's keys into
    ranges for separate workgroups; needs a float32 workspace of `latent_decode_workspace_floats` floats. sink float32
    [heads]: exp(sink_a) more in head a's denominator (no key, no value, not scaled)."""
    _need(sink is None or (sink.dtype == torch.float32 and sink.is_contiguous() and sink.numel() == heads), "sink must be float32 [heads]")
    page, K = keys.shape[2], keys.shape[3]
    Lp = values.shape[2]
    nq, wq, ldq = _rows(q, "q")
    no, wo, ldo = _rows(out, "out")
    _need(wq == heads * K and wo == heads * Lp and no >= n_seqs and nq >= n_seqs, "latent_decode q/out shapes do not agree")
    _need(out.dtype == q.dtype == keys.dtype == values.dtype, "attention operand types differ")
    _need(keys.dim() == 4 and keys.shape[1] == 1 and keys.is_contiguous() and values.is_contiguous()
          and tuple(values.shape) == (keys.shape[0], 1, Lp, page), "keys [pages, 1, page, K], values [pages, 1, latent_dev, page]")
    _need(K % 16 == 0 and K <= 256 and Lp % 16 == 0 and 16 <= Lp <= 240 and Lp <= K and page % 4 == 0, "unsupported sizes")
    _need(block_table.dim() == 2 and block_table.stride(1) == 1 and block_table.shape[0] >= n_seqs, "block_table must be 2-D")
    _need(q_start.numel() >= n_seqs + 1 and kv_len.numel() >= n_seqs, "sequence metadata is too short")
    ws_ptr, ws_floats = None, 0
    if splits > 1:
        _need(workspace is not None and workspace.dtype == torch.float32, "split attention needs a float32 workspace")
        ws_ptr, ws_floats = _dev(workspace), workspace.numel()
    check(library().tw_latent_decode(dtype_id(q.dtype), _dev(q), ldq, _dev(keys), _dev(values),
                                     _dev(block_table, torch.int32, "block_table"), block_table.stride(0),
                                     _dev(q_start, torch.int32, "q_start"), _dev(kv_len, torch.int32, "kv_len"), int(n_seqs),
                                     _dev(out), ldo, ws_ptr, ws_floats, int(heads), K, Lp, page, float(scale), int(splits),
                                     _dev(sink) if sink is not None else None, _stream()), "latent_decode")
    return out


def latent_gather(keys, block_table, kv_len, kv_page_start, seq0, n_seqs, own_pages, rows, own_table):
    """The cached key rows of sequences seq0 .. seq0 + n_seqs - 1 from their pages into pages of their own, sequence after
    sequence (own page kv_page_start[s] - kv_page_start[seq0] + b holds block b of sequence s; places past a sequence's
    end are zeros), and those pages' numbers into own_table[s, b]. keys [pages, 1, page, K]; rows [own_pages * page, K]."""
    page, K = keys.shape[2], keys.shape[3]
    _need(keys.dim() == 4 and keys.shape[1] == 1 and keys.is_contiguous(), "keys must be contiguous [pages, 1, page, K]")
    _need(rows.is_contiguous() and tuple(rows.shape) == (own_pages * page, K) and rows.dtype == keys.dtype, "rows must be [own_pages * page, K]")
    _need(own_table.dtype == torch.int32 and own_table.dim() == 2 and own_table.stride(1) == 1 and own_table.shape[0] >= seq0 + n_seqs,
          "own_table must be int32 [sequences, blocks]")
    _need(block_table.dim() == 2 and block_table.stride(1) == 1 and block_table.shape[0] >= seq0 + n_seqs
          and own_table.shape[1] >= block_table.shape[1], "block_table must be 2-D and own_table as wide")
    _need(kv_len.numel() >= seq0 + n_seqs and kv_page_start.numel() >= seq0 + n_seqs + 1, "sequence metadata is too short")
    check(library().tw_latent_gather(dtype_id(keys.dtype), _dev(keys), _dev(block_table, torch.int32, "block_table"),
                                     block_table.stride(0), _dev(kv_len, torch.int32, "kv_len"),
                                     _dev(kv_page_start, torch.int32, "kv_page_start"), _dev(rows), _dev(own_table),
                                     own_table.stride(0), int(seq0), int(n_seqs), int(own_pages), page, K, _stream()), "latent_gather")


def latent_expand_store(up, rows, latent_dev, keys, values, heads, dim, rot, value_dim):
    """keys[page, a, place] = [up[row, a * dim : (a + 1) * dim] | rows[row, latent_dev : latent_dev + rot] | zeros] and
    values[page, a, :, place] = [up[row, heads * dim + a * value_dim ...] | zeros] for row = page * page_size + place.
    keys [own_pages, heads, page, hd]; values [own_pages, heads, hd, page]."""
    n, wu, ld_up = _rows(up, "up")
    own_pages, H, page, hd = keys.shape
    _need(H == heads and keys.is_contiguous() and values.is_contiguous() and tuple(values.shape) == (own_pages, H, hd, page)
          and keys.dtype == up.dtype == rows.dtype == values.dtype, "keys [own_pages, heads, page, hd], values [own_pages, heads, hd, page]")
    _need(n == own_pages * page and wu == heads * (dim + value_dim) and rows.is_contiguous() and rows.shape[0] == n
          and rows.shape[1] >= latent_dev + rot and hd >= max(dim + rot, value_dim), "latent_expand_store shapes do not agree")
    check(library().tw_latent_expand_store(dtype_id(up.dtype), _dev(up), ld_up, _dev(rows), rows.shape[1], int(latent_dev), _dev(keys),
                                           _dev(values), own_pages, heads, int(dim), int(rot), int(value_dim), hd, page, _stream()),
          "latent_expand_store")


def head_linear(x, x_stride, weight, out, out_stride):
    """out[n, a * out_stride + o] = sum_i x[n, a * x_stride + i] * weight[a, o, i]; weight [heads, No, Ni] of x's type
    (Ni a multiple of 16 bytes, No of 4); out has x's type; float32 sums, one rounding."""
    n, wx, ldx = _rows(x, "x")
    no, wo, ldo = _rows(out, "out")
    heads, n_out, n_in = weight.shape
    epf = 16 // x.element_size()
    _need(weight.is_contiguous() and weight.dtype == x.dtype == out.dtype and no == n, "head_linear operand types or rows differ")
    _need(n_in % epf == 0 and n_out % 4 == 0 and x_stride % epf == 0 and ldx % epf == 0 and x.data_ptr() % 16 == 0,
          "head_linear: inputs must be 16-byte aligned and Ni a multiple of 16 bytes, No of 4")
    _need((heads - 1) * x_stride + n_in <= wx and (heads - 1) * out_stride + n_out <= wo and out_stride >= n_out,
          "head_linear: the heads exceed the rows")
    _need((ldo * out.element_size()) % 8 == 0 and (out_stride * out.element_size()) % 8 == 0 and out.data_ptr() % 8 == 0,
          "head_linear: output rows and heads must be 8-byte aligned")
    check(library().tw_head_linear(dtype_id(x.dtype), _dev(x), ldx, int(x_stride), _dev(weight), _dev(out), ldo, int(out_stride),
                                   n, heads, n_in, n_out, _stream()), "head_linear")
    return out


# ---- retention ------------------------------------------------------------------------------------------------

def retention_workspace_floats(n_seqs, max_q_len, heads, key_dev, value_dev):
    """float32 scratch the chunked retention kernel needs for portions of up to max_q_len tokens (0: none): long
    portions are cut into segments for separate workgroups, which leave their partial states there."""
    return int(library().tw_retention_workspace_floats(int(n_seqs), int(max_q_len), int(heads), int(key_dev), int(value_dev)))


def retention(proj, q_col, k_col, v_col, cos, sin, decay, state, q_start, state_slots, seq0, n_seqs, out, k_scale,
              max_q_len=0, workspace=None):
    """S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head for sequences seq0 .. seq0 + n_seqs - 1, from and to
    state float32 [requests, H, Dp, Ep]. q, k (unrotated) and v are columns of proj (head h at col + h * Dp, or
    + h * Ep); they are rotated with cos/sin float32 [n, rot / 2] (None: no rotation) and k then multiplied by k_scale.
    out float32 [n, H * Ep]. max_q_len > 0: the kernel that walks a sequence's rows in chunks on the matrix unit, for
    portions of up to that many tokens (with a workspace of `retention_workspace_floats` floats where that is not
    zero); 0: the one that walks them token by token (one-token steps)."""
    n, width, ld = _rows(proj, "proj")
    _need(state.dim() == 4 and state.is_contiguous() and state.dtype == torch.float32, "state must be float32 [requests, H, Dp, Ep]")
    H, Dp, Ep = state.shape[1:]
    rot = 0
    if cos is not None:
        rot = 2 * cos.shape[1]
        _need(tuple(cos.shape) == (n, rot // 2) and tuple(sin.shape) == (n, rot // 2) and cos.is_contiguous() and sin.is_contiguous()
              and cos.dtype == torch.float32, "rotary tables must be float32 [n, rot / 2]")
    _need(Dp % 16 == 0 and Dp <= 256 and rot <= Dp, "key heads are multiples of 16 up to 256 on the device")
    _need(max(q_col, k_col) + H * Dp <= width and v_col + H * Ep <= width, "q, k or v exceed the projection's row")
    no, wo, ldo = _rows(out, "out")
    _need(no == n and wo == H * Ep and out.dtype == torch.float32, "out must be float32 [n, H * Ep]")
    _need(decay.numel() == H and decay.dtype == torch.float32, "one float32 decay per head")
    _need(seq0 >= 0 and q_start.numel() >= seq0 + n_seqs + 1 and state_slots.numel() >= seq0 + n_seqs, "sequence metadata is too short")
    _need(ldo % 4 == 0 and out.data_ptr() % 16 == 0, "out rows must be 16-byte aligned")
    need = retention_workspace_floats(n_seqs, max_q_len, H, Dp, Ep) if max_q_len > 0 else 0
    if need:
        _need(workspace is not None and workspace.dtype == torch.float32 and workspace.is_contiguous() and workspace.numel() >= need,
              "long portions need a float32 workspace of retention_workspace_floats floats")
    check(library().tw_retention(dtype_id(proj.dtype), _dev(proj), ld, int(q_col), int(k_col), int(v_col),
                                 _dev(cos) if rot else None, _dev(sin) if rot else None, rot, _dev(decay), _dev(state),
                                 _dev(q_start, torch.int32, "q_start"), _dev(state_slots, torch.int32, "state_slots"),
                                 _dev(out), ldo, int(seq0), int(n_seqs), int(max_q_len), H, Dp, Ep, float(k_scale),
                                 _dev(workspace) if need else None, workspace.numel() if need else 0, _stream()),
          "retention")
    return out


def unit_gate(o, gate, out, heads, value_dim, value_dev, eps):
    """out[n, h, e] = o[n, h, e] / sqrt(mean_e o^2 + eps) * silu(gate[n, h, e]) over each head's value_dim real
    elements (heads value_dev apart, tails zero); o float32, gate and out of the compute type."""
    n, wo, ld_o = _rows(o, "o")
    ng, wg, ld_g = _rows(gate, "gate")
    nn, wn, ld_n = _rows(out, "out")
    _need(o.dtype == torch.float32 and gate.dtype == out.dtype, "o is float32; gate and out share the compute type")
    _need(ng == n and nn == n and min(wo, wg, wn) >= heads * value_dev and value_dim <= value_dev, "unit_gate shapes do not agree")
    check(library().tw_unit_gate(dtype_id(out.dtype), _dev(o), ld_o, _dev(gate), ld_g, _dev(out), ld_n, n, heads, int(value_dim),
                                 int(value_dev), float(eps), _stream()), "unit_gate")
    return out


# ---- what the Rufusun design added ------------------------------------------------------------------------------

def swish_limited_mul(gate_up, out, limit):
    """out[n, i] = g' * sigmoid(1.702 g') * (u' + 1) with g' = min(gate_up[n, i], limit), u' = clamp(gate_up[n, inter + i],
    -limit, limit): the limited swish where gate and up rows cannot be interleaved for the product's epilogue."""
    n, inter = out.shape
    _need(gate_up.is_contiguous() and out.is_contiguous() and tuple(gate_up.shape) == (n, 2 * inter) and gate_up.dtype == out.dtype,
          "swish_limited_mul takes contiguous [n, 2 * inter] and [n, inter] of one type")
    check(library().tw_swish_limited_mul(dtype_id(out.dtype), _dev(gate_up), _dev(out), n, inter, float(limit), _stream()),
          "swish_limited_mul")
    return out


def rmsnorm_pair(x, weight1, eps, out1, weight2=None, out2=None):
    """out1 = x * rsqrt(mean(x^2) + eps) * weight1 and, if asked for, out2 = the same rows times weight2: two norms of
    the same float32 rows from one pass (the weights are float32 and hold every factor, a stored offset included)."""
    _need(x.dim() == 2 and x.is_contiguous() and x.dtype == torch.float32, "rmsnorm_pair input must be contiguous float32 [n, hidden]")
    n, hidden = x.shape
    _need((weight2 is None) == (out2 is None), "a second weight and a second output come together")
    for w, o in ((weight1, out1), (weight2, out2)):
        if w is not None:
            _need(w.numel() == hidden and w.is_contiguous() and o.is_contiguous() and tuple(o.shape) == (n, hidden)
                  and o.dtype == out1.dtype, "rmsnorm_pair weights are [hidden], outputs contiguous [n, hidden] of one type")
    check(library().tw_rmsnorm_pair(dtype_id(out1.dtype), _dev(x), _dev(weight1, torch.float32, "weight1"),
                                    _dev(weight2, torch.float32, "weight2") if weight2 is not None else None, _dev(out1),
                                    _dev(out2) if out2 is not None else None, n, hidden, float(eps), _stream()), "rmsnorm_pair")
    return out1, out2


def scale_values(x, factor):
    """x *= factor in place (contiguous float32)."""
    _need(x.is_contiguous() and x.dtype == torch.float32, "scale_values takes a contiguous float32 tensor")
    check(library().tw_scale_values(_dev(x), x.numel(), float(factor), _stream()), "scale_values")
    return x


def delta_key_extent(dim):
    """Elements a column of the delta rule's state holds on the device: the key size rounded up to a multiple of 4."""
    return (int(dim) + 3) // 4 * 4


def delta_rule(qkv, q_col, k_col, v_col, ab, b_col, a_col, A_log, dt_bias, state, q_start, state_slots, seq0, n_seqs, out,
               kv_heads, dim, q_scale, max_q_len=1):
    """The gated delta rule over sequences seq0 .. seq0 + n_seqs - 1, from and to state float32
    [requests, H, E, Dk] (a column of S is contiguous; Dk = delta_key_extent(dim)):

        q~ = unit(q) * q_scale, k~ = unit(k) (unit: x / sqrt(sum x^2 + 1e-6)), beta = sigmoid(b),
        g = exp(-exp(A_log) * softplus(a + dt_bias));  S <- g S;  u = beta (v - S^T k~);  S <- S + k~ u^T;  o = S^T q~

    qkv float32 [n, .]: q of key head j at q_col + j * dim, k at k_col + j * dim, v of head h at v_col + h * E;
    ab float32 [n, .]: b of head h at b_col + h, a at a_col + h; value head h reads key head h // (H / kv_heads).
    out float32 [n, H * E]. max_q_len: the most tokens a sequence brings (an upper bound will do). Up to a few tokens
    a sequence the tokens are walked one by one; beyond, chunks of 16 tokens are solved at once (the same sums in another
    order: a triangular system a chunk in place of a chain of updates)."""
    n, wq, ld_qkv = _rows(qkv, "qkv")
    na, wa, ld_ab = _rows(ab, "ab")
    _need(qkv.dtype == torch.float32 and ab.dtype == torch.float32 and na == n, "the delta rule reads float32 rows")
    _need(state.dim() == 4 and state.is_contiguous() and state.dtype == torch.float32, "state must be float32 [requests, H, E, Dk]")
    H, E, Dk = state.shape[1:]
    G, D = int(kv_heads), int(dim)
    _need(G > 0 and H % G == 0 and 0 < D <= 256 and Dk == delta_key_extent(D), "the delta rule takes key sizes up to 256, H a multiple of the key heads")
    _need(min(q_col, k_col, v_col, a_col, b_col) >= 0 and max(q_col, k_col) + G * D <= wq and v_col + H * E <= wq
          and max(a_col, b_col) + H <= wa, "q, k, v, a or b exceed their rows")
    no, wo, ldo = _rows(out, "out")
    _need(no == n and wo == H * E and out.dtype == torch.float32, "out must be float32 [n, H * E]")
    _need(A_log.numel() == H and dt_bias.numel() == H and A_log.dtype == torch.float32 and dt_bias.dtype == torch.float32,
          "one float32 A_log and dt_bias per head")
    _need(seq0 >= 0 and q_start.numel() >= seq0 + n_seqs + 1 and state_slots.numel() >= seq0 + n_seqs, "sequence metadata is too short")
    check(library().tw_delta_rule(_dev(qkv), ld_qkv, int(q_col), int(k_col), int(v_col), _dev(ab), ld_ab, int(b_col), int(a_col),
                                  _dev(A_log), _dev(dt_bias), _dev(state), _dev(q_start, torch.int32, "q_start"),
                                  _dev(state_slots, torch.int32, "state_slots"), _dev(out), ldo, int(seq0), int(n_seqs),
                                  max(1, int(max_q_len)), H, G, D, E, Dk, float(q_scale), _stream()), "delta_rule")
    return out


def head_norm_gate(o, gate, weight, out, heads, value_dim, eps, gate_activation="silu"):
    """out[n, h, e] = o[n, h, e] / sqrt(mean_e o^2 + eps) * weight[e] * act(gate[n, h, e]); o and gate float32, weight
    float32 [value_dim] shared by the heads or [heads * value_dim] with one vector a head, out of the compute type;
    act the SiLU or ("sigmoid") the sigmoid of the gate."""
    _need(gate_activation in ("silu", "sigmoid"), "the gate passes 'silu' or 'sigmoid'")
    n, wo, ld_o = _rows(o, "o")
    ng, wg, ld_g = _rows(gate, "gate")
    nn, wn, ld_n = _rows(out, "out")
    _need(o.dtype == torch.float32 and gate.dtype == torch.float32, "o and gate are float32")
    _need(ng == n and nn == n and min(wo, wg, wn) >= heads * value_dim and weight.numel() in (value_dim, heads * value_dim)
          and weight.is_contiguous(), "head_norm_gate shapes do not agree")
    per_head = 1 if (weight.numel() == heads * value_dim and heads > 1) else 0
    check(library().tw_head_norm_gate(dtype_id(out.dtype), _dev(o), ld_o, _dev(gate), ld_g, _dev(weight, torch.float32, "weight"),
                                      _dev(out), ld_n, n, int(heads), int(value_dim), float(eps), per_head,
                                      1 if gate_activation == "sigmoid" else 0, _stream()), "head_norm_gate")
    return out


MOE_MAX_EXPERTS = 1024


MOE_WEIGHTS = {"sigmoid": 0, "softmax_chosen": 1}


def moe_route(h, router, top, ids, weights, bias=None, weighting="sigmoid"):
    """ids[n, top], weights[n, top]: per row of h the `top` experts with the largest router logits router @ h + bias
    (float32 products of h's values as they are; the lowest index wins a tie), and per chosen logit its sigmoid or
    ("softmax_chosen") its share of the softmax over the chosen logits alone."""
    _need(weighting in MOE_WEIGHTS, "a router's weights are 'sigmoid' or 'softmax_chosen'")
    n, C, ld_h = _rows(h, "h")
    X = router.shape[0]
    _need(router.dtype == torch.float32 and router.is_contiguous() and tuple(router.shape) == (X, C), "the router is float32 [experts, C]")
    _need(0 < top <= X <= MOE_MAX_EXPERTS, f"1 to {MOE_MAX_EXPERTS} experts, of which at most all are chosen")
    _need(ids.is_contiguous() and weights.is_contiguous() and tuple(ids.shape) == (n, top) and tuple(weights.shape) == (n, top),
          "ids and weights are [n, top]")
    _need(bias is None or (bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == X), "the router's bias is float32 [experts]")
    check(library().tw_moe_route(dtype_id(h.dtype), _dev(h), ld_h, _dev(router), _dev(bias) if bias is not None else None,
                                 MOE_WEIGHTS[weighting], n, C, X, int(top), _dev(ids, torch.int32, "ids"),
                                 _dev(weights, torch.float32, "weights"), _stream()), "moe_route")
    return ids, weights


def moe_capacity(items, experts):
    """Rows the experts' order can take for ITEMS (token, choice) pairs: every expert's share rounded up to 16 rows."""
    return int(library().tw_moe_capacity(int(items), int(experts)))


def moe_pad(size):
    """A size the grouped products take as their K: rounded up to a multiple of 32 (zeros fill the rest)."""
    return (int(size) + 31) // 32 * 32


def moe_blocked(w):
    """Stacked matrices [X, N, K] (K a multiple of 32) in the order the grouped products read them: rows padded with zeros
    to a multiple of 16, then [X, N16 / 16, K / (4 EPF), piece 0..3, row 0..15, EPF] (EPF: the elements of 16 bytes),
    returned as [X, N16, K]: a wave's load of one fragment is 1 KB of consecutive memory."""
    X, N, K = w.shape
    epf = 16 // w.element_size()
    _need(K % 32 == 0, "K must be padded to a multiple of 32")
    N16 = (N + 15) // 16 * 16
    if N16 != N:
        w = torch.cat([w, w.new_zeros(X, N16 - N, K)], 1)
    return w.reshape(X, N16 // 16, 16, K // (4 * epf), 4, epf).permute(0, 1, 3, 4, 2, 5).contiguous().reshape(X, N16, K)


MOE_KINDS = {"swish_limited": 0, "gelu": 1}


def moe_experts(h, ids, weights, gate, up, down, limit, x, scratch, kind="swish_limited", accumulate=True, more=None):
    """kind "gelu" (gate None): x[n] (+)= sum over a row's chosen experts e of weights_e * down_e(gelu(up_e h[n])), the exact
    gelu; accumulate=False writes x instead of adding to it; more: float32 [splits, n, C] partial sums of something that
    belongs to the same result (a shared expert's last product), added up here as well. kind "swish_limited": x[n] += sum over a row's chosen experts e of down_e(glu(gate_e y, up_e y)), y = round(weights * h[n]), glu the
    limited swish with LIMIT. gate, up [X, Fd, Cd], down [X, C16, Fd] in h's type, zero padded (Fd, Cd: `moe_pad` of the
    sizes, C16: C rounded up to 16) and laid out by `moe_blocked`. scratch(tag, shape, dtype) hands out the step's scratch tensors."""
    n, C, ld_h = _rows(h, "h")
    top = ids.shape[1]
    _need(kind in MOE_KINDS and (gate is None) == (kind == "gelu"), "experts are 'swish_limited' (with a gate) or 'gelu' (without)")
    X, Fd, Cd = up.shape
    _need((gate is None or (gate.is_contiguous() and gate.dtype == h.dtype and tuple(gate.shape) == (X, Fd, Cd)))
          and up.is_contiguous() and down.is_contiguous() and up.dtype == down.dtype == h.dtype,
          "the experts' matrices are contiguous and of h's type")
    _need(tuple(up.shape) == (X, Fd, Cd) and tuple(down.shape) == (X, (C + 15) // 16 * 16, Fd) and Cd == moe_pad(C) and Fd % 32 == 0,
          "the experts' matrices are [X, Fd, Cd] and [X, C16, Fd]")
    _need(ids.is_contiguous() and weights.is_contiguous() and tuple(ids.shape) == (n, top) and tuple(weights.shape) == (n, top),
          "ids and weights are [n, top]")
    nx, cx, ld_x = _rows(x, "x")
    _need(nx == n and cx == C and x.dtype == torch.float32, "x must be float32 [n, C]")
    if more is not None:
        _need(more.dim() == 3 and more.is_contiguous() and tuple(more.shape[1:]) == (n, C) and more.dtype == torch.float32,
              "more must be float32 [splits, n, C]")
    capacity = moe_capacity(n * top, X)
    pos = scratch("moe.pos", (n * top,), torch.int32)
    src_item = scratch("moe.src", (capacity,), torch.int32)
    tile_expert = scratch("moe.tiles", (capacity // 16,), torch.int32)
    xs = scratch("moe.xs", (capacity, Cd), h.dtype)
    act = scratch("moe.act", (capacity, Fd), h.dtype)
    ys = scratch("moe.ys", (capacity, C), torch.float32)
    check(library().tw_moe_experts(dtype_id(h.dtype), _dev(h), ld_h, _dev(ids, torch.int32, "ids"),
                                   _dev(weights, torch.float32, "weights"), n, top, X, _dev(gate) if gate is not None else None,
                                   _dev(up), _dev(down), C, Cd, Fd,
                                   float(limit), _dev(pos), _dev(src_item), _dev(tile_expert), _dev(xs), _dev(act), _dev(ys),
                                   capacity, _dev(x), ld_x, MOE_KINDS[kind], 1 if accumulate else 0,
                                   _dev(more) if more is not None else None, more.shape[0] if more is not None else 0,
                                   _stream()), "moe_experts")
    return x


# ---- a norm on a sublayer's result, output gates, convolved and normed queries and keys, the mLSTM ------------------------

def add_normed(x, weight, eps, mult=1.0, y=None, add=None, out=None):
    """x <- x + mult * weight * unit(y), unit(v) = v / sqrt(mean(v^2) + eps); x float32 [n, hidden] in place.

    y: float32 [n, hidden] (rows may be strided), or add: float32 [splits, n, hidden] partial sums added up here;
    out: the new x once more, rounded to its type (the compute type)."""
    _need(x.dim() == 2 and x.is_contiguous() and x.dtype == torch.float32, "add_normed: x must be contiguous float32 [n, hidden]")
    n, hidden = x.shape
    _need(weight.numel() == hidden and weight.dtype == torch.float32 and weight.is_contiguous(), "the norm weight must be float32 [hidden]")
    _need((y is None) != (add is None), "either y or partial sums")
    ldy, splits, stride = 0, 0, 0
    if y is not None:
        ny, cy, ldy = _rows(y, "y")
        _need((ny, cy) == (n, hidden) and y.dtype == torch.float32, "y must be float32 [n, hidden]")
    else:
        _need(add.dim() == 3 and add.is_contiguous() and tuple(add.shape[1:]) == (n, hidden) and add.dtype == torch.float32,
              "partial sums must be float32 [splits, n, hidden]")
        splits, stride = add.shape[0], n * hidden
    out_dtype = F32
    if out is not None:
        _need(out.is_contiguous() and tuple(out.shape) == (n, hidden), "out must be contiguous [n, hidden]")
        out_dtype = dtype_id(out.dtype)
    check(library().tw_add_normed(out_dtype, _dev(x), _dev(y) if y is not None else None, ldy,
                                  _dev(add) if add is not None else None, splits, stride, _dev(weight),
                                  _dev(out) if out is not None else None, n, hidden, float(mult), float(eps), _stream()),
          "add_normed")
    return x


def activation(x, kind, partial=None):
    """x <- act(x) in place (rows may be strided), act "relu_squared" or "gelu" (the exact one); with PARTIAL (float32
    [splits, n, cols], split-K sums of the product before) x <- act(sum of the splits) instead, rounded once."""
    _need(kind in LINEAR_ACTIVATIONS, "an activation is 'relu_squared' or 'gelu'")
    n, cols, ld = _rows(x, "x")
    splits = 0
    if partial is not None:
        _need(partial.dim() == 3 and partial.is_contiguous() and tuple(partial.shape[1:]) == (n, cols)
              and partial.dtype == torch.float32, "partial sums must be float32 [splits, n, cols]")
        splits = partial.shape[0]
    check(library().tw_activation(dtype_id(x.dtype), _dev(x), ld, n, cols, _dev(partial) if partial is not None else None,
                                  splits, LINEAR_ACTIVATIONS[kind], _stream()), "activation")
    return x


def sigmoid_gate(out, gate):
    """out <- out * sigmoid(gate), element by element; gate float32 or of out's type, rows of both may be strided."""
    n, cols, ld_out = _rows(out, "out")
    ng, cg, ld_g = _rows(gate, "gate")
    _need((ng, cg) == (n, cols) and gate.dtype in (torch.float32, out.dtype), "gate must be [n, cols], float32 or of out's type")
    check(library().tw_sigmoid_gate(dtype_id(out.dtype), _dev(out), ld_out, _dev(gate), ld_g,
                                    1 if gate.dtype == torch.float32 else 0, n, cols, _stream()), "sigmoid_gate")
    return out


def softcap_values(x, cap):
    """x <- cap * tanh(x / cap) over a contiguous float32 tensor, in place."""
    _need(x.dtype == torch.float32 and x.is_contiguous() and float(cap) > 0, "softcap_values takes contiguous float32 and a positive cap")
    check(library().tw_softcap_values(_dev(x), x.numel(), float(cap), _stream()), "softcap_values")
    return x


def qk_finish(src, q_col, k_col, q_weight, k_weight, cos, sin, q_out, keys, values, slots, q_heads, kv_heads, dim, rot,
              eps, adjacent=False):
    """Per token: q <- rotate(q_weight * unit(q)), k <- rotate(k_weight * unit(k)), v = k as it came; unit over the WHOLE
    row of q (q_heads * dim elements at src[:, q_col:]) and of k (kv_heads * dim at k_col), rotation of the first `rot`
    elements of every head. src float32. q_out [n, q_heads * dim_dev] in the compute type (tails of zeros); keys
    [pages, kv_heads, page, dim_dev], values [pages, kv_heads, dim_dev, page]; slots[n] the token's page slot (-1: not stored)."""
    n, width, ld = _rows(src, "src")
    nq, wq, ld_q = _rows(q_out, "q_out")
    page, dim_dev = keys.shape[2], keys.shape[3]
    _need(src.dtype == torch.float32 and nq == n and wq == q_heads * dim_dev, "qk_finish: src float32, q_out [n, q_heads * dim_dev]")
    _need(keys.is_contiguous() and values.is_contiguous() and keys.dtype == values.dtype == q_out.dtype
          and tuple(keys.shape[1:]) == (kv_heads, page, dim_dev) and tuple(values.shape) == (keys.shape[0], kv_heads, dim_dev, page),
          "keys [pages, kv_heads, page, dim_dev], values [pages, kv_heads, dim_dev, page] of q_out's type")
    _need(q_weight.dtype == torch.float32 and q_weight.is_contiguous() and q_weight.numel() == q_heads * dim
          and k_weight.dtype == torch.float32 and k_weight.is_contiguous() and k_weight.numel() == kv_heads * dim,
          "the norms' weights are float32 over the whole rows")
    _need(q_col + q_heads * dim <= width and k_col + kv_heads * dim <= width and slots.numel() == n and dim <= dim_dev,
          "qk_finish: columns exceed the rows, or not one slot per row")
    if rot:
        _need(cos is not None and cos.dtype == torch.float32 and cos.is_contiguous() and tuple(cos.shape) == (n, rot // 2)
              and tuple(sin.shape) == (n, rot // 2), "cos and sin are float32 [n, rot / 2]")
    check(library().tw_qk_finish(dtype_id(q_out.dtype), _dev(src), ld, int(q_col), int(k_col), _dev(q_weight), _dev(k_weight),
                                 _dev(cos) if rot else None, _dev(sin) if rot else None, _dev(q_out), ld_q, _dev(keys),
                                 _dev(values), _dev(slots, torch.int32, "slots"), n, int(q_heads), int(kv_heads), int(dim),
                                 dim_dev, int(rot), 1 if adjacent else 0, page, float(eps), _stream()), "qk_finish")
    return q_out


MLSTM_WALK_TOKENS = 4          # sequences with up to this many tokens in a step are walked token by token


def mlstm(proj, q_col, k_col, v_col, i_col, f_col, i_bias, f_bias, S, n_state, m_state, q_start, state_slots, phase, seq0,
          n_seqs, out, heads, dim, value_dim, q_scale, cap, walk, first_row=None):
    """The mLSTM's matrix memory over sequences seq0 .. seq0 + n_seqs - 1 of a step. proj float32 rows with q, k
    (heads * dim each), v (heads * value_dim) and the two gates' raw values (heads each) at the given columns; i_bias,
    f_bias float32 [heads]. S float32 [requests, heads, value_dev, dim_dev], n_state [requests, 2, heads, dim_dev], m_state
    [requests, 2, heads] (copy phase[s] is read, the other written). out float32 [rows, heads * value_dim]: S^T q over its
    denominator. walk: token by token (steps of a few tokens a sequence), else chunks of 16 on the matrix unit; then
    first_row, if given, says that the launch's sequences own the rows from there to proj's last: their gates are formed
    first by a kernel of their own, IN PLACE of the raw values in proj."""
    n, width, ld = _rows(proj, "proj")
    no, wo, ld_out = _rows(out, "out")
    dim_dev, value_dev = (dim + 15) // 16 * 16, (value_dim + 15) // 16 * 16
    _need(proj.dtype == torch.float32 and out.dtype == torch.float32 and no == n and wo == heads * value_dim, "mlstm: float32 rows")
    _need(1 <= dim <= 256, "the mLSTM kernels take key sizes up to 256")
    _need(max(q_col, k_col) + heads * dim <= width and v_col + heads * value_dim <= width and max(i_col, f_col) + heads <= width,
          "mlstm: columns exceed the rows")
    requests = S.shape[0]
    for t, shape, name in ((S, (requests, heads, value_dev, dim_dev), "S"), (n_state, (requests, 2, heads, dim_dev), "n"),
                           (m_state, (requests, 2, heads), "m")):
        _need(t.dtype == torch.float32 and t.is_contiguous() and tuple(t.shape) == shape, f"mlstm: state {name} must be float32 {shape}")
    for t, name in ((i_bias, "i_bias"), (f_bias, "f_bias")):
        _need(t.dtype == torch.float32 and t.is_contiguous() and t.numel() == heads, f"{name} must be float32 [heads]")
    _need(q_start.numel() >= seq0 + n_seqs + 1 and state_slots.numel() >= seq0 + n_seqs and phase.numel() >= seq0 + n_seqs,
          "sequence metadata is too short")
    check(library().tw_mlstm(_dev(proj), ld, int(q_col), int(k_col), int(v_col), int(i_col), int(f_col), _dev(i_bias), _dev(f_bias),
                             _dev(S), _dev(n_state), _dev(m_state), _dev(q_start, torch.int32, "q_start"),
                             _dev(state_slots, torch.int32, "state_slots"), _dev(phase, torch.int32, "phase"), int(seq0),
                             int(n_seqs), _dev(out), ld_out, int(heads), int(dim), int(value_dim), float(q_scale), float(cap),
                             1 if walk else 0, -1 if (walk or first_row is None) else int(first_row), n, _stream()), "mlstm")
    return out
