"""Python faces of the HIP kernels.  Each function checks on the host that the
operands have the shapes, dtypes and layout its kernel and grid assume (a
mismatch is an error here, never a wrong result or a fault on the device), then
launches on torch's current stream.  Tensors must live on the GPU; there is no
CPU path."""
import ctypes

import numpy as np

import torch

from . import library

PAGE = 64                       # tokens per cache page (csrc/common.h)
PREFILL_MIXED_TILES = 64        # prefill_tile_order mixes the sequences of a step up to this many tiles
MAX_HEAD_DIM = 1024             # of the float32-arithmetic attention kernels (above 256: a latent attention's one wide head)
MFMA_HEAD_DIMS = tuple(range(16, 129, 16))   # head sizes of the matrix-core attention kernels (others: float32 arithmetic)

_DT = {torch.float32: 0, torch.bfloat16: 1}

# set by tests to run the float32-arithmetic kernels also for bfloat16 storage
FORCE_SIMPLE = False


def dtype_code(dtype):
    try:
        return _DT[dtype]
    except KeyError:
        raise TypeError("unsupported dtype %s (float32 or bfloat16)" % dtype) from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current stream's handle (a launch asks for it: the short way, where torch has one)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _need(t, name, dtype=None, shape=None):
    """The address of a tensor after the checks every kernel argument gets; the first lines are the way of an
    argument that passes them (a step of a short prompt is a few hundred launches that the host has to keep up with)."""
    try:
        fine = t.is_cuda and t.is_contiguous() and (dtype is None or t.dtype == dtype)
    except AttributeError:
        fine = False
    if fine:
        if shape is None:
            return t.data_ptr()
        have = t.shape
        if len(have) == len(shape):
            for s, d in zip(shape, have):
                if s is not None and s != d:
                    break
            else:
                return t.data_ptr()
    if not isinstance(t, torch.Tensor):
        raise TypeError("%s: expected a tensor" % name)
    if not t.is_cuda:
        raise RuntimeError("%s: the HIP kernels need GPU tensors (got %s); there is no CPU path" % (name, t.device))
    if not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)
    if dtype is not None and t.dtype != dtype:
        raise TypeError("%s: expected %s, got %s" % (name, dtype, t.dtype))
    if shape is not None:
        if t.dim() != len(shape) or any(s is not None and s != d for s, d in zip(shape, t.shape)):
            raise ValueError("%s: expected shape %s, got %s" % (name, list(shape), list(t.shape)))
    return t.data_ptr()


def _opt(t, name, dtype=None, shape=None):
    return None if t is None else _need(t, name, dtype, shape)


def embed(table, tokens, out):
    """out[t] = float(table[tokens[t]]); a negative token gives zeros."""
    V, D = table.shape
    T = tokens.shape[0]
    p_table = _need(table, "table")
    code = dtype_code(table.dtype)
    p_tok = _need(tokens, "tokens", torch.int32, (T,))
    p_out = _need(out, "out", torch.float32, (T, D))
    library.check(library.lib().yalm_embed(p_table, code, p_tok, p_out, T, D, V, _stream()), "embed")
    return out


def embed_sinusoid(table, tokens, positions, freq, scale, out):
    """out[t] = float(table[tokens[t]]) * scale + (freq given) the sinusoidal vector of positions[t]: entry 2i is
    sin(p freq[i]), entry 2i + 1 the cosine; freq float64 [ceil(D / 2)] on the device.  A negative token gives zeros."""
    V, D = table.shape
    T = tokens.shape[0]
    p_freq = None if freq is None else _need(freq, "freq", torch.float64, ((D + 1) // 2,))
    p_pos = None if freq is None else _need(positions, "positions", torch.int32, (T,))
    library.check(library.lib().yalm_embed_sinusoid(
        _need(table, "table"), dtype_code(table.dtype), _need(tokens, "tokens", torch.int32, (T,)), p_pos, p_freq,
        float(scale), _need(out, "out", torch.float32, (T, D)), T, D, V, _stream()), "embed_sinusoid")
    return out


def rmsnorm(x, weight, out, eps, row_index=None):
    """out[r] = x[row_index[r] or r] * rsqrt(mean(x^2) + eps) * weight."""
    D = x.shape[-1]
    R = out.shape[0]
    p_x = _need(x, "x", torch.float32, (None, D))
    p_w = _need(weight, "weight", None, (D,))
    p_o = _need(out, "out", None, (R, D))
    p_i = _opt(row_index, "row_index", torch.int32, (R,))
    if row_index is None and x.shape[0] < R:
        raise ValueError("rmsnorm: %d rows wanted of %d" % (R, x.shape[0]))
    library.check(library.lib().yalm_rmsnorm(p_x, p_w, dtype_code(weight.dtype), p_o, dtype_code(out.dtype), p_i, R, D,
                                             float(eps), _stream()), "rmsnorm")
    return out


EPI_STORE_F32, EPI_STORE, EPI_ADD_F32, EPI_GATED = 0, 1, 2, 3
EPI_GATED_GELU = 5          # as EPI_GATED with the reference's gelu (tanh form) in silu's place (src/infer.cpp:189-195)
GATED = (EPI_GATED, EPI_GATED_GELU)


GEMM_SPLIT_MAX = 16          # most K slices a GEMM uses, given the workspace


def gemm_workspace_floats(M, N, K):
    """Floats of scratch with which a bfloat16 gemm splits K across workgroups: 17..64 rows (to 128 with K a multiple of 64), and
    more rows than that while the output's tiles alone would leave most of the chip idle."""
    if 16 < M <= 64 or (M <= 128 and K % 64 == 0):
        return GEMM_SPLIT_MAX * M * N
    if M > 64:
        return int(library.lib().yalm_gemm_bf16_dma_workspace(M, N, K))
    return 0


def gemm(a, w, out, epilogue, hidden=0, workspace=None, scale_from=None):
    """out = a[M,K] @ w[N,K]^T with float32 accumulation and one of four epilogues:
    EPI_STORE_F32 (float32 out), EPI_STORE (out in a's dtype), EPI_ADD_F32
    (float32 out += product), EPI_GATED (w = gate/up rows interleaved in blocks of
    16; out[M, hidden] = silu(gate) * up in a's dtype; EPI_GATED_GELU: gelu(gate) * up).  workspace: float32 scratch of
    gemm_workspace_floats(M, N, K) elements, with which small batches split K.
    scale_from = (ss float32 [M, parts], eps), 17..128 bfloat16 rows only (can_add_emit): a was emitted by
    gemm_add_emit, and the sums are scaled by rsqrt(sum(ss[m]) / K + eps) per row before the epilogue."""
    M, K = a.shape
    N = w.shape[0]
    dt = a.dtype
    p_a = _need(a, "a", dt, (M, K))
    p_w = _need(w, "w", dt, (N, K))
    if epilogue in GATED:
        if hidden <= 0 or N != 32 * ((hidden + 15) // 16):
            raise ValueError("gated gemm: weight rows %d do not match hidden %d" % (N, hidden))
        p_o = _need(out, "out", dt, (M, hidden))
    elif epilogue == EPI_STORE:
        p_o = _need(out, "out", dt, (M, N))
    elif epilogue in (EPI_STORE_F32, EPI_ADD_F32):
        p_o = _need(out, "out", torch.float32, (M, N))
    else:
        raise ValueError("unknown epilogue %r" % (epilogue,))
    p_ws, n_ws = None, 0
    if workspace is not None:
        p_ws, n_ws = _need(workspace, "workspace", torch.float32), workspace.numel()
    if scale_from is not None:
        ss, eps = scale_from
        if dt != torch.bfloat16:
            raise TypeError("gemm: a row scale goes with bfloat16 activations")
        p_ss = _need(ss, "ss", torch.float32, (M, None))
        library.check(library.lib().yalm_gemm_scaled(p_a, p_w, p_o, p_ws, n_ws, M, N, K, epilogue, hidden, p_ss,
                                                     ss.shape[1], float(eps), _stream()), "gemm with a row scale")
        return out
    library.check(library.lib().yalm_gemm(p_a, p_w, p_o, p_ws, n_ws, M, N, K, dtype_code(dt), epilogue, hidden,
                                          1 if FORCE_SIMPLE else 0, _stream()), "gemm")
    return out


FUSED_NORM_MAX_ROWS = 8


def can_fuse_norm(M, K, dtype):
    """Whether gemm_norm / gemm_norm_qkv_rope take this shape (else: rmsnorm, then gemm)."""
    return dtype == torch.bfloat16 and 1 <= M <= FUSED_NORM_MAX_ROWS and K % 8 == 0 and \
        M * (K + 8) * 2 <= 72 * 1024 and not FORCE_SIMPLE


def gemm_norm(x, norm_w, eps, w, out, epilogue, hidden=0):
    """out = epilogue(rmsnorm(x, norm_w, eps) @ w^T) for at most 16 rows of the float32
    residual stream x; w bfloat16 [N, K], norm_w float32 [K]; EPI_STORE_F32, EPI_GATED or EPI_GATED_GELU.
    (Shapes: see can_fuse_norm.)"""
    M, K = x.shape
    N = w.shape[0]
    p_x = _need(x, "x", torch.float32, (M, K))
    p_n = _need(norm_w, "norm_w", torch.float32, (K,))
    p_w = _need(w, "w", torch.bfloat16, (N, K))
    if epilogue in GATED:
        if hidden <= 0 or N != 32 * ((hidden + 15) // 16):
            raise ValueError("gated gemm: weight rows %d do not match hidden %d" % (N, hidden))
        p_o = _need(out, "out", torch.bfloat16, (M, hidden))
    elif epilogue == EPI_STORE_F32:
        p_o = _need(out, "out", torch.float32, (M, N))
    else:
        raise ValueError("gemm_norm: epilogue %r is not offered" % (epilogue,))
    library.check(library.lib().yalm_gemm_norm(p_x, p_n, float(eps), p_w, p_o, M, N, K, epilogue, hidden, _stream()),
                  "gemm_norm")
    return out


PAGE_ROWS, PAGE_BLOCKS = 0, 1


def page_layout(head_dim):
    """How keys and values lie inside a cache page of a head: PAGE_ROWS (keys [row][element], values
    [element][row]) or, for head sizes that are multiples of 32, PAGE_BLOCKS (keys [element // 32][place of the
    row in the order the matrix-core decode attention takes rows][element % 32], values [row // 32][element]
    [row % 32]), in which every load instruction of that kernel reads 1 KB of consecutive bytes.  The tensors'
    shapes stay [pages, heads, PAGE, head_dim] and [pages, heads, head_dim, PAGE] either way."""
    return PAGE_BLOCKS if head_dim % 32 == 0 else PAGE_ROWS


def _layout(layout, head_dim):
    layout = page_layout(head_dim) if layout is None else int(layout)
    if layout not in (PAGE_ROWS, PAGE_BLOCKS) or (layout == PAGE_BLOCKS and head_dim % 32):
        raise ValueError("page layout %r does not fit head_dim %d" % (layout, head_dim))
    return layout


def gemm_norm_qkv_rope(x, norm_w, eps, wqkv, q_out, k_pages, v_pages, block_table, ring_pages, tok_pos, seq_slot,
                       cos_sin, n_heads, n_kv_heads, head_dim, rotary_dim, layout=None):
    """A decode step's rmsnorm + q/k/v projection + rotation + cache write in one kernel
    (row m is sequence m; see rope_kv_write for the operands)."""
    _check_heads(n_heads, n_kv_heads, head_dim)
    if head_dim % 16:
        raise ValueError("gemm_norm_qkv_rope needs a head_dim that is a multiple of 16")
    M, K = x.shape
    Q, KV = n_heads * head_dim, n_kv_heads * head_dim
    p_x = _need(x, "x", torch.float32, (M, K))
    p_n = _need(norm_w, "norm_w", torch.float32, (K,))
    p_w = _need(wqkv, "wqkv", torch.bfloat16, (Q + 2 * KV, K))
    p_q = _need(q_out, "q_out", torch.bfloat16, (M, Q))
    n_pages = k_pages.shape[0]
    p_kp = _need(k_pages, "k_pages", torch.bfloat16, (n_pages, n_kv_heads, PAGE, head_dim))
    p_vp = _need(v_pages, "v_pages", torch.bfloat16, (n_pages, n_kv_heads, head_dim, PAGE))
    p_bt = _need(block_table, "block_table", torch.int32, (None, None))
    stride = block_table.shape[1]
    if ring_pages <= 0 or ring_pages > stride:
        raise ValueError("ring_pages %d does not fit the block table (%d columns)" % (ring_pages, stride))
    p_tp = _need(tok_pos, "tok_pos", torch.int32, (M,))
    p_ss = _need(seq_slot, "seq_slot", torch.int32, (M,))
    n_pos, p_cs = 0, None
    if cos_sin is not None:
        n_pos = cos_sin.shape[0]
        p_cs = _need(cos_sin, "cos_sin", torch.float32, (n_pos, rotary_dim // 2, 2))
    else:
        rotary_dim = 0
    library.check(library.lib().yalm_gemm_norm_qkv_rope(
        p_x, p_n, float(eps), p_w, p_q, p_kp, p_vp, p_bt, stride, ring_pages, p_tp, p_ss, p_cs, n_pos, M, K, n_heads,
        n_kv_heads, head_dim, rotary_dim, n_pages, _layout(layout, head_dim), _stream()), "gemm_norm_qkv_rope")


CHAIN_MAX_ROWS = 16


def can_chain(M, K, dtype):
    """Whether gemm_chain / gemm_chain_qkv_rope take this shape."""
    return dtype == torch.bfloat16 and 1 <= M <= CHAIN_MAX_ROWS and K % 8 == 0 and not FORCE_SIMPLE


def can_add_norm(M, K, dtype):
    """Whether gemm_add_norm takes this shape (the batches that gemm_chain leaves out)."""
    if dtype != torch.bfloat16 or FORCE_SIMPLE or M <= CHAIN_MAX_ROWS:
        return False
    return K % 8 == 0 if M <= 64 else K % 64 == 0


def fused_workspace_floats(M, N, K):
    """Floats of scratch for gemm_add_norm and gemm_partial: what lets the GEMM split K as it likes,
    and room for one whole product at least."""
    return max(gemm_workspace_floats(M, N, K), M * N)


def gemm_add_norm(a, w, x, norm_w, eps, h_out, workspace):
    """x float32 [M, N] += a[M, K] @ w[N, K]^T for more than 16 bfloat16 rows (more than 64: K a multiple
    of 64), and h_out bfloat16 [M, N] = RMSNorm(x_new) with the weights norm_w (float32 [N]): the residual add and the next norm in one.
    workspace: float32 scratch of gemm_workspace_floats(M, N, K) elements."""
    M, K = a.shape
    N = w.shape[0]
    p_a = _need(a, "a", torch.bfloat16, (M, K))
    p_w = _need(w, "w", torch.bfloat16, (N, K))
    p_x = _need(x, "x", torch.float32, (M, N))
    p_nw = _need(norm_w, "norm_w", torch.float32, (N,))
    p_h = _need(h_out, "h_out", torch.bfloat16, (M, N))
    if workspace is None or workspace.numel() < M * N:
        raise ValueError("gemm_add_norm needs a workspace of at least M * N floats")
    p_ws = _need(workspace, "workspace", torch.float32, None)
    library.check(library.lib().yalm_gemm_add_norm(p_a, p_w, p_x, p_ws, workspace.numel(), M, N, K, p_nw, float(eps),
                                                   p_h, _stream()), "gemm_add_norm")
    return h_out


def can_add_emit(M, K, dtype):
    """Whether gemm_add_emit takes this shape, and gemm / gemm_partial a row scale for M rows: batches beyond the
    norm chain of gemm_chain (16 rows) up to 128 rows."""
    return can_add_norm(M, K, dtype) and M <= 128


def gemm_add_emit_parts(N):
    """Columns of the partial sums of squares that gemm_add_emit leaves for rows of N columns."""
    return library.lib().yalm_gemm_add_emit_parts(int(N))


def gemm_add_emit(a, w, x, norm_w, xn_out, ss_out, workspace):
    """x float32 [M, N] += a[M, K] @ w[N, K]^T (shapes as gemm_add_norm), xn_out bfloat16 [M, N] = x_new * norm_w and
    ss_out float32 [M, gemm_add_emit_parts(N)] = partial sums of squares of x_new: the next norm prepared but not
    finished; its consumer scales its own sums (gemm / gemm_partial with scale_from)."""
    M, K = a.shape
    N = w.shape[0]
    p_a = _need(a, "a", torch.bfloat16, (M, K))
    p_w = _need(w, "w", torch.bfloat16, (N, K))
    p_x = _need(x, "x", torch.float32, (M, N))
    p_nw = _need(norm_w, "norm_w", torch.float32, (N,))
    p_xn = _need(xn_out, "xn_out", torch.bfloat16, (M, N))
    p_ss = _need(ss_out, "ss_out", torch.float32, (M, gemm_add_emit_parts(N)))
    if workspace is None or workspace.numel() < M * N:
        raise ValueError("gemm_add_emit needs a workspace of at least M * N floats")
    p_ws = _need(workspace, "workspace", torch.float32, None)
    library.check(library.lib().yalm_gemm_add_emit(p_a, p_w, p_x, p_ws, workspace.numel(), M, N, K, p_nw, p_xn, p_ss,
                                                   _stream()), "gemm_add_emit")
    return xn_out


def can_gemm_partial(M, K, dtype):
    """True if gemm_partial takes the shape (more than 16 rows of bfloat16; more than 64: K a multiple of 64)."""
    return can_add_norm(M, K, dtype)


def gemm_partial(a, w, workspace, scale_from=None):
    """The K slices of a[M,K] @ w[N,K]^T, more than 16 rows of bfloat16 (more than 64: K a multiple of
    64), left unadded in `workspace`
    ([slices][M][N] float32, flat; gemm_workspace_floats(M, N, K) elements let it split as it likes).
    Returns the number of slices, for a consumer that adds them (rope_kv_write).  scale_from as in gemm
    (every slice is scaled)."""
    M, K = a.shape
    N = w.shape[0]
    p_a = _need(a, "a", torch.bfloat16, (M, K))
    p_w = _need(w, "w", torch.bfloat16, (N, K))
    p_ws = _need(workspace, "workspace", torch.float32, (None,))
    if workspace.numel() < M * N:
        raise ValueError("workspace holds %d floats, at least %d are needed" % (workspace.numel(), M * N))
    slices = ctypes.c_int(0)
    if scale_from is not None:
        ss, eps = scale_from
        p_ss = _need(ss, "ss", torch.float32, (M, None))
        library.check(library.lib().yalm_gemm_partial_scaled(p_a, p_w, p_ws, workspace.numel(), M, N, K,
                                                             ctypes.byref(slices), p_ss, ss.shape[1], float(eps),
                                                             _stream()), "gemm_partial with a row scale")
        return slices.value
    library.check(library.lib().yalm_gemm_partial(p_a, p_w, p_ws, workspace.numel(), M, N, K, ctypes.byref(slices),
                                                  _stream()), "gemm_partial")
    return slices.value


def gemm_chain_parts(N):
    """Columns of the partial sums of squares that a producer with N output columns emits."""
    return library.lib().yalm_gemm_chain_parts(int(N))


def gemm_chain(x, w, out, epilogue, hidden=0, scale_from=None, emit=None):
    """Decode GEMM (bfloat16; at most CHAIN_MAX_ROWS rows: beyond that the per-workgroup sum of the
    partial sums costs more than a norm kernel) that chains norms.
    scale_from = (ss float32 [M, parts], eps): x was emitted as bfloat16(residual * norm weight) and
    the product is scaled by rsqrt(sum(ss[m]) / K + eps) per row.
    emit = (norm_w float32 [N], xn bfloat16 [M, N], ss float32 [M, gemm_chain_parts(N)]), with
    EPI_ADD_F32 only: also writes xn = bfloat16(out_new * norm_w) and the partial sums of squares."""
    M, K = x.shape
    N = w.shape[0]
    p_x = _need(x, "x", torch.bfloat16, (M, K))
    p_w = _need(w, "w", torch.bfloat16, (N, K))
    if epilogue in GATED:
        if hidden <= 0 or N != 32 * ((hidden + 15) // 16):
            raise ValueError("gated gemm: weight rows %d do not match hidden %d" % (N, hidden))
        p_o = _need(out, "out", torch.bfloat16, (M, hidden))
    elif epilogue in (EPI_STORE_F32, EPI_ADD_F32):
        p_o = _need(out, "out", torch.float32, (M, N))
    else:
        raise ValueError("gemm_chain: epilogue %r is not offered" % (epilogue,))
    p_ss, n_parts, eps = None, 0, 0.0
    if scale_from is not None:
        ss, eps = scale_from
        n_parts = ss.shape[1]
        p_ss = _need(ss, "ss", torch.float32, (M, n_parts))
    p_nw = p_xn = p_es = None
    if emit is not None:
        if epilogue != EPI_ADD_F32:
            raise ValueError("gemm_chain: only the residual-add epilogue emits")
        nw, xn, es = emit
        p_nw = _need(nw, "emit norm_w", torch.float32, (N,))
        p_xn = _need(xn, "emit xn", torch.bfloat16, (M, N))
        p_es = _need(es, "emit ss", torch.float32, (M, gemm_chain_parts(N)))
    library.check(library.lib().yalm_gemm_chain(p_x, p_w, p_o, M, N, K, epilogue, hidden, p_ss, n_parts, float(eps),
                                                p_nw, p_xn, p_es, _stream()), "gemm_chain")
    return out


def gemm_chain_qkv_rope(xn, scale_from, wqkv, q_out, k_pages, v_pages, block_table, ring_pages, tok_pos, seq_slot,
                        cos_sin, n_heads, n_kv_heads, head_dim, rotary_dim, layout=None):
    """gemm_norm_qkv_rope for activations a producer emitted (see gemm_chain)."""
    _check_heads(n_heads, n_kv_heads, head_dim)
    if head_dim % 16:
        raise ValueError("gemm_chain_qkv_rope needs a head_dim that is a multiple of 16")
    M, K = xn.shape
    Q, KV = n_heads * head_dim, n_kv_heads * head_dim
    ss, eps = scale_from
    n_parts = ss.shape[1]
    p_x = _need(xn, "xn", torch.bfloat16, (M, K))
    p_ss = _need(ss, "ss", torch.float32, (M, n_parts))
    p_w = _need(wqkv, "wqkv", torch.bfloat16, (Q + 2 * KV, K))
    p_q = _need(q_out, "q_out", torch.bfloat16, (M, Q))
    n_pages = k_pages.shape[0]
    p_kp = _need(k_pages, "k_pages", torch.bfloat16, (n_pages, n_kv_heads, PAGE, head_dim))
    p_vp = _need(v_pages, "v_pages", torch.bfloat16, (n_pages, n_kv_heads, head_dim, PAGE))
    p_bt = _need(block_table, "block_table", torch.int32, (None, None))
    stride = block_table.shape[1]
    if ring_pages <= 0 or ring_pages > stride:
        raise ValueError("ring_pages %d does not fit the block table (%d columns)" % (ring_pages, stride))
    p_tp = _need(tok_pos, "tok_pos", torch.int32, (M,))
    p_sl = _need(seq_slot, "seq_slot", torch.int32, (M,))
    n_pos, p_cs = 0, None
    if cos_sin is not None:
        n_pos = cos_sin.shape[0]
        p_cs = _need(cos_sin, "cos_sin", torch.float32, (n_pos, rotary_dim // 2, 2))
    else:
        rotary_dim = 0
    library.check(library.lib().yalm_gemm_chain_qkv_rope(
        p_x, p_ss, n_parts, float(eps), p_w, p_q, p_kp, p_vp, p_bt, stride, ring_pages, p_tp, p_sl, p_cs, n_pos, M, K,
        n_heads, n_kv_heads, head_dim, rotary_dim, n_pages, _layout(layout, head_dim), _stream()),
        "gemm_chain_qkv_rope")


def _check_heads(n_heads, n_kv_heads, head_dim):
    if n_heads % n_kv_heads != 0:
        raise ValueError("n_heads %d is no multiple of n_kv_heads %d" % (n_heads, n_kv_heads))
    if head_dim % 2 != 0 or head_dim <= 0 or head_dim > MAX_HEAD_DIM:
        raise ValueError("head_dim %d is not supported (even, at most %d)" % (head_dim, MAX_HEAD_DIM))


def rope_kv_write(qkv, q_out, k_stage, v_stage, seq_tile0, k_pages, v_pages, block_table, ring_pages, tok_seq, tok_pos,
                  seq_slot, seq_len, cos_sin, n_heads, n_kv_heads, head_dim, rotary_dim, slices=1, layout=None):
    """Rotates q and k by the angles of `cos_sin` at each token's position, writes q in
    q_out's dtype, k and v into the staging area (page format, tile seq_tile0[sequence] +
    position // PAGE) if one is given, and into the pages of the cache if given.
    slices > 1: qkv is the flat scratch of gemm_partial, [slices][T][q + 2 kv] float32, and the
    slices are added while they are read."""
    _check_heads(n_heads, n_kv_heads, head_dim)
    T = q_out.shape[0]
    Q, KV = n_heads * head_dim, n_kv_heads * head_dim
    dt = q_out.dtype
    if slices == 1 and qkv.dim() == 2:
        p_qkv = _need(qkv, "qkv", torch.float32, (T, Q + 2 * KV))
    else:
        p_qkv = _need(qkv, "qkv", torch.float32, (None,))
        if slices < 1 or qkv.numel() < slices * T * (Q + 2 * KV):
            raise ValueError("qkv holds %d floats, %d slices of %d rows need %d"
                             % (qkv.numel(), slices, T, slices * T * (Q + 2 * KV)))
    p_q = _need(q_out, "q_out", dt, (T, Q))
    B = seq_slot.shape[0]
    p_ks = p_vs = p_t0 = None
    if k_stage is not None:
        n_tiles = k_stage.shape[0]
        p_ks = _need(k_stage, "k_stage", dt, (n_tiles, n_kv_heads, PAGE, head_dim))
        p_vs = _need(v_stage, "v_stage", dt, (n_tiles, n_kv_heads, head_dim, PAGE))
        p_t0 = _need(seq_tile0, "seq_tile0", torch.int32, (B + 1,))
    n_pages = 0
    p_kp = p_vp = p_bt = None
    stride = 0
    if k_pages is not None:
        n_pages = k_pages.shape[0]
        p_kp = _need(k_pages, "k_pages", dt, (n_pages, n_kv_heads, PAGE, head_dim))
        p_vp = _need(v_pages, "v_pages", dt, (n_pages, n_kv_heads, head_dim, PAGE))
        p_bt = _need(block_table, "block_table", torch.int32, (None, None))
        stride = block_table.shape[1]
        if ring_pages <= 0 or ring_pages > stride:
            raise ValueError("ring_pages %d does not fit the block table (%d columns)" % (ring_pages, stride))
    p_ts = _need(tok_seq, "tok_seq", torch.int32, (T,))
    p_tp = _need(tok_pos, "tok_pos", torch.int32, (T,))
    p_ss = _need(seq_slot, "seq_slot", torch.int32, (B,))
    p_sl = _need(seq_len, "seq_len", torch.int32, (B,))
    n_pos = 0
    p_cs = None
    if cos_sin is not None:
        if rotary_dim % 2 != 0 or rotary_dim > head_dim or rotary_dim <= 0:
            raise ValueError("rotary_dim %d does not fit head_dim %d" % (rotary_dim, head_dim))
        n_pos = cos_sin.shape[0]
        p_cs = _need(cos_sin, "cos_sin", torch.float32, (n_pos, rotary_dim // 2, 2))
    else:
        rotary_dim = 0
    library.check(library.lib().yalm_rope_kv_write(
        p_qkv, p_q, p_ks, p_vs, p_t0, p_kp, p_vp, p_bt, stride, max(ring_pages, 1), p_ts, p_tp, p_ss, p_sl, p_cs,
        n_pos, T, n_heads, n_kv_heads, head_dim, rotary_dim, n_pages, _layout(layout, head_dim), int(slices),
        dtype_code(dt), _stream()), "rope_kv_write")


def rope_kv_write_tiles(qkv, q_out, k_stage, v_stage, cu_seqlens, seq_tile0, k_pages, v_pages, block_table, ring_pages,
                        seq_slot, seq_len, cos_sin, n_heads, n_kv_heads, head_dim, rotary_dim, slices=1, layout=None):
    """rope_kv_write for a step of whole prompts (every sequence from position 0), a page-shaped
    tile of 64 positions at a time.  False if the kernel refuses the head size (the caller then
    uses rope_kv_write).  slices as in rope_kv_write."""
    _check_heads(n_heads, n_kv_heads, head_dim)
    T = q_out.shape[0]
    Q, KV = n_heads * head_dim, n_kv_heads * head_dim
    dt = q_out.dtype
    if head_dim * (PAGE + 8) * dt.itemsize > 64 * 1024:
        return False
    B = seq_slot.shape[0]
    n_tiles = k_stage.shape[0]
    if slices == 1 and qkv.dim() == 2:
        p_qkv = _need(qkv, "qkv", torch.float32, (T, Q + 2 * KV))
    else:
        p_qkv = _need(qkv, "qkv", torch.float32, (None,))
        if slices < 1 or qkv.numel() < slices * T * (Q + 2 * KV):
            raise ValueError("qkv holds %d floats, %d slices of %d rows need %d"
                             % (qkv.numel(), slices, T, slices * T * (Q + 2 * KV)))
    p_q = _need(q_out, "q_out", dt, (T, Q))
    p_ks = _need(k_stage, "k_stage", dt, (n_tiles, n_kv_heads, PAGE, head_dim))
    p_vs = _need(v_stage, "v_stage", dt, (n_tiles, n_kv_heads, head_dim, PAGE))
    p_cu = _need(cu_seqlens, "cu_seqlens", torch.int32, (B + 1,))
    p_t0 = _need(seq_tile0, "seq_tile0", torch.int32, (B + 1,))
    n_pages, stride = 0, 0
    p_kp = p_vp = p_bt = None
    if k_pages is not None:
        n_pages = k_pages.shape[0]
        p_kp = _need(k_pages, "k_pages", dt, (n_pages, n_kv_heads, PAGE, head_dim))
        p_vp = _need(v_pages, "v_pages", dt, (n_pages, n_kv_heads, head_dim, PAGE))
        p_bt = _need(block_table, "block_table", torch.int32, (None, None))
        stride = block_table.shape[1]
        if ring_pages <= 0 or ring_pages > stride:
            raise ValueError("ring_pages %d does not fit the block table (%d columns)" % (ring_pages, stride))
    p_ss = _need(seq_slot, "seq_slot", torch.int32, (B,))
    p_sl = _need(seq_len, "seq_len", torch.int32, (B,))
    n_pos = 0
    p_cs = None
    if cos_sin is not None:
        if rotary_dim % 2 != 0 or rotary_dim > head_dim or rotary_dim <= 0:
            raise ValueError("rotary_dim %d does not fit head_dim %d" % (rotary_dim, head_dim))
        n_pos = cos_sin.shape[0]
        p_cs = _need(cos_sin, "cos_sin", torch.float32, (n_pos, rotary_dim // 2, 2))
    else:
        rotary_dim = 0
    library.check(library.lib().yalm_rope_kv_write_tiles(
        p_qkv, p_q, p_ks, p_vs, p_cu, p_t0, p_kp, p_vp, p_bt, stride, max(ring_pages, 1), p_ss, p_sl, p_cs, n_pos, T, B,
        n_tiles, n_heads, n_kv_heads, head_dim, rotary_dim, n_pages, _layout(layout, head_dim), int(slices),
        dtype_code(dt), _stream()), "rope_kv_write_tiles")
    return True


def prefill_tile_order(n_tokens):
    """The order in which attn_prefill should take the tiles of a step whose sequences bring
    n_tokens tokens each: every second 64-token tile of a sequence (its workgroup covers the
    next one too).  A short step (at most 4,096 tokens with their padding) has the tiles that
    see the most keys first, whatever their sequence; a longer one goes sequence by sequence,
    the longest first and each from its end, so that the workgroups running together read the
    same keys (measured: 8 prompts of 2,048 tokens lose 4 % when their tiles are mixed).  A numpy
    int32 array for the host side of the step's metadata."""
    n_tiles = [(n + PAGE - 1) // PAGE for n in n_tokens]
    first = np.concatenate([[0], np.cumsum(n_tiles)])
    tiles, work = [], []
    for b in sorted(range(len(n_tiles)), key=lambda b: -n_tiles[b]):
        for tq in range((n_tiles[b] - 1) // 2 * 2, -1, -2):
            tiles.append(int(first[b]) + tq)
            work.append(min(tq + 2, n_tiles[b]))
    tiles = np.asarray(tiles, dtype=np.int32)
    if int(first[-1]) <= PREFILL_MIXED_TILES:
        tiles = tiles[np.argsort(-np.asarray(work, dtype=np.int64), kind="stable")]
    return tiles


def _bias(score_bias, n_heads):
    """(address, distances) of a score bias: float32 [n_heads, n] on the device, added to every score (scaled by
    1/sqrt(head_dim) already) as score_bias[head, min(query position - key position, n - 1)]; None: no bias.  What a
    position encoding that is no rotation needs (a slope per head times the distance, a learned table)."""
    if score_bias is None:
        return None, 0
    n = score_bias.shape[-1]
    return _need(score_bias, "score_bias", torch.float32, (n_heads, n)), n


def _log_distance(log_distance, n_heads):
    """(address of a, address of b) of a term that grows with the logarithm of the distance: log_distance = (a, b), two
    float32 [n_heads] on the device, adds -a[head] * ln(1 + b[head] * (query position - key position)) to every score
    (behind the cap); None: no such term."""
    if log_distance is None:
        return None, None
    a, b = log_distance
    return _need(a, "log_distance a", torch.float32, (n_heads,)), _need(b, "log_distance b", torch.float32, (n_heads,))


def _shape(softcap, sink_logit, n_heads, slopes=None):
    """(cap, address of the sink logits, address of the slopes): softcap > 0 replaces every scaled score s by softcap
    tanh(s / softcap) before the score bias; sink_logit, float32 [n_heads] on the device, puts one more term exp(sink_logit[head]) into the
    softmax's denominator, a term to which no key and no row of values belongs; slopes, float32 [n_heads] on the device, adds
    -slopes[head] * (query position - key position) to every score (what a score_bias table of slope times distance
    would add, without the table)."""
    cap = float(softcap or 0.0)
    if cap < 0.0:
        raise ValueError("a score cap must be positive (0: none)")
    return cap, _opt(sink_logit, "sink_logit", torch.float32, (n_heads,)), _opt(slopes, "slopes", torch.float32, (n_heads,))


def attn_prefill(q, k_stage, v_stage, out, cu_seqlens, seq_tile0, tok_seq, tok_pos, n_heads, n_kv_heads, head_dim,
                 window, tile_order=None, lse=None, out_f32=None, score_bias=None, softcap=0.0, sink_logit=None, slopes=None,
                 block=0, log_distance=None):
    """Causal (and windowed) attention of packed sequences that start at position 0, over
    the keys and values that rope_kv_write staged for this step.  tile_order (device int32,
    from prefill_tile_order) only changes the order of the work.  lse (float32 [T, n_heads], optional)
    receives the logarithm of every query's sum of exp(score), for attn_sink_mix; out_f32 (float32 [T, n_heads *
    head_dim], optional) the result before it is rounded to out's dtype, for the same.  score_bias: see _bias;
    softcap, sink_logit: see _shape; log_distance: see _log_distance.  block > 0: a query sees only the keys of its own block of `block` positions
    (blocks counted from position 0 of its sequence), beside what the window says."""
    if block < 0:
        raise ValueError("a block of positions has a positive size (0: none)")
    _check_heads(n_heads, n_kv_heads, head_dim)
    T = q.shape[0]
    dt = q.dtype
    B = cu_seqlens.shape[0] - 1
    n_tiles = k_stage.shape[0]
    p_q = _need(q, "q", dt, (T, n_heads * head_dim))
    p_k = _need(k_stage, "k_stage", dt, (n_tiles, n_kv_heads, PAGE, head_dim))
    p_v = _need(v_stage, "v_stage", dt, (n_tiles, n_kv_heads, head_dim, PAGE))
    p_o = _need(out, "out", dt, (T, n_heads * head_dim))
    p_cu = _need(cu_seqlens, "cu_seqlens", torch.int32, (B + 1,))
    p_t0 = _need(seq_tile0, "seq_tile0", torch.int32, (B + 1,))
    p_ts = _need(tok_seq, "tok_seq", torch.int32, (T,))
    p_tp = _need(tok_pos, "tok_pos", torch.int32, (T,))
    p_or, n_order = None, 0
    if tile_order is not None:
        n_order = tile_order.shape[0]
        p_or = _need(tile_order, "tile_order", torch.int32, (n_order,))
    p_lse = None if lse is None else _need(lse, "lse", torch.float32, (T, n_heads))
    p_o32 = _opt(out_f32, "out_f32", torch.float32, (T, n_heads * head_dim))
    library.check(library.lib().yalm_attn_prefill_lse(p_q, p_k, p_v, p_o, p_o32, p_lse, p_cu, p_t0, p_ts, p_tp, p_or, n_order,
                                                      T, B, n_tiles, n_heads, n_kv_heads, head_dim, int(window),
                                                      dtype_code(dt), 1 if FORCE_SIMPLE else 0,
                                                      *_bias(score_bias, n_heads), *_shape(softcap, sink_logit, n_heads, slopes),
                                                      int(block), *_log_distance(log_distance, n_heads), _stream()),
                  "attn_prefill")
    return out


def attn_decode_workspace_floats(B, n_heads, head_dim, n_splits):
    return library.lib().yalm_attn_decode_workspace(B, n_heads, head_dim, n_splits) // 4


def attn_decode(q, k_pages, v_pages, block_table, ring_pages, seq_slot, seq_len, out, partial, n_heads, n_kv_heads,
                head_dim, window, n_splits, lse=None, sinks=None, layout=None, step_max_len=None, seq_order=None,
                score_bias=None, softcap=0.0, sink_logit=None, slopes=None, block=0, log_distance=None):
    """One query per sequence over the cache pages (laid out as `layout` says, default page_layout(head_dim));
    seq_len counts the new key.  lse as in attn_prefill.  step_max_len (int32 [1] on the device, optional): the
    length of the step's longest sequence, with which sequences of unequal lengths are cut into splits of equal
    size; seq_order (int32 [B] on the device, a permutation of the rows, optional): the order in which the
    workgroups take the rows (both change the division of the work and no result).  score_bias: see _bias; softcap,
    sink_logit: see _shape; block: see attn_prefill (none of these with sinks).
    sinks = (sink_k, sink_v [slots, n_kv_heads, n_sinks, head_dim], cos_sin or None, rotary_dim, store):
    the attention sinks that a query's window no longer covers are taken in where the splits are merged
    (their keys turned by max(0, position - window - n_sinks + 1) positions with the table cos_sin); with
    `store` a token at one of its sequence's first n_sinks positions stores its key and value there."""
    _check_heads(n_heads, n_kv_heads, head_dim)
    B = q.shape[0]
    dt = q.dtype
    n_pages = k_pages.shape[0]
    p_q = _need(q, "q", dt, (B, n_heads * head_dim))
    p_kp = _need(k_pages, "k_pages", dt, (n_pages, n_kv_heads, PAGE, head_dim))
    p_vp = _need(v_pages, "v_pages", dt, (n_pages, n_kv_heads, head_dim, PAGE))
    p_bt = _need(block_table, "block_table", torch.int32, (None, None))
    stride = block_table.shape[1]
    if ring_pages <= 0 or ring_pages > stride:
        raise ValueError("ring_pages %d does not fit the block table (%d columns)" % (ring_pages, stride))
    p_ss = _need(seq_slot, "seq_slot", torch.int32, (B,))
    p_sl = _need(seq_len, "seq_len", torch.int32, (B,))
    p_o = _need(out, "out", dt, (B, n_heads * head_dim))
    need = attn_decode_workspace_floats(B, n_heads, head_dim, n_splits)
    p_w = _need(partial, "partial", torch.float32)
    if partial.numel() < need:
        raise ValueError("attn_decode workspace too small: %d floats, %d needed" % (partial.numel(), need))
    force = 1 if FORCE_SIMPLE else 0
    p_max = _opt(step_max_len, "step_max_len", torch.int32, (1,))
    p_ord = _opt(seq_order, "seq_order", torch.int32, (B,))
    if sinks is None:
        p_lse = None if lse is None else _need(lse, "lse", torch.float32, (B, n_heads))
        library.check(library.lib().yalm_attn_decode_lse(
            p_q, p_kp, p_vp, p_bt, stride, ring_pages, p_ss, p_sl, p_o, p_lse, p_w, B, n_heads, n_kv_heads, head_dim,
            int(window), int(n_splits), n_pages, _layout(layout, head_dim), dtype_code(dt), force, p_max, p_ord,
            *_bias(score_bias, n_heads), *_shape(softcap, sink_logit, n_heads, slopes), int(block),
            *_log_distance(log_distance, n_heads), _stream()), "attn_decode")
        return out
    if lse is not None:
        raise ValueError("attn_decode leaves no lse when it takes the sinks in itself")
    if score_bias is not None or softcap or sink_logit is not None or slopes is not None or block or log_distance is not None:
        raise ValueError("attention sinks are scored without a score bias, a cap or a sink logit: they do not go together")
    sink_k, sink_v, cos_sin, rotary_dim, store = sinks
    n_slots, _, n_sinks, _ = sink_k.shape
    if window < n_sinks:
        raise ValueError("a window of %d is narrower than the %d sinks beside it" % (window, n_sinks))
    if block_table.shape[0] < n_slots:
        raise ValueError("the block table has %d rows for %d slots" % (block_table.shape[0], n_slots))
    n_pos, p_cs = 0, None
    if cos_sin is not None and rotary_dim > 0:
        n_pos = cos_sin.shape[0]
        p_cs = _need(cos_sin, "cos_sin", torch.float32, (n_pos, rotary_dim // 2, 2))
    library.check(library.lib().yalm_attn_decode_sinks(
        p_q, p_kp, p_vp, p_bt, stride, ring_pages, p_ss, p_sl, p_o, p_w,
        _need(sink_k, "sink_k", dt, (n_slots, n_kv_heads, n_sinks, head_dim)),
        _need(sink_v, "sink_v", dt, (n_slots, n_kv_heads, n_sinks, head_dim)), 1 if store else 0, p_cs, n_pos, n_slots,
        int(rotary_dim) if p_cs is not None else 0, n_sinks, B, n_heads, n_kv_heads, head_dim, int(window),
        int(n_splits), n_pages, _layout(layout, head_dim), dtype_code(dt), force, p_max, p_ord, _stream()),
        "attn_decode with sinks")
    return out


MAX_SINKS = 16


def sink_store(k_stage, v_stage, seq_tile0, seq_slot, seq_len, sink_k, sink_v):
    """A step of whole prompts: copies the keys and values of positions < min(n_sinks, seq_len) from the
    staging area (sequence b's first tile is seq_tile0[b]) into the per-slot store sink_k, sink_v
    [slots, n_kv_heads, n_sinks, head_dim]."""
    n_slots, n_kv_heads, n_sinks, head_dim = sink_k.shape
    dt = sink_k.dtype
    n_tiles = k_stage.shape[0]
    B = seq_slot.shape[0]
    library.check(library.lib().yalm_sink_store(
        _need(k_stage, "k_stage", dt, (n_tiles, n_kv_heads, PAGE, head_dim)),
        _need(v_stage, "v_stage", dt, (n_tiles, n_kv_heads, head_dim, PAGE)),
        _need(seq_tile0, "seq_tile0", torch.int32, (B + 1,)), _need(seq_slot, "seq_slot", torch.int32, (B,)),
        _need(seq_len, "seq_len", torch.int32, (B,)), _need(sink_k, "sink_k", dt),
        _need(sink_v, "sink_v", dt, (n_slots, n_kv_heads, n_sinks, head_dim)), B, n_tiles, n_slots, n_kv_heads,
        head_dim, n_sinks, dtype_code(dt), _stream()), "sink_store")


def attn_sink_mix(q, out, lse, sink_k, sink_v, tok_seq, tok_pos, seq_slot, cos_sin, n_heads, rotary_dim, window,
                  src_f32=None):
    """A step of whole prompts: adds the attention sinks that the window no longer covers to the attention
    result `out` (in place): for the token at position p the sinks j < min(n_sinks, p - window + 1), their
    keys turned by max(0, p - window - n_sinks + 1) positions with the table cos_sin (None: not turned).
    lse is what attn_prefill left for these queries; src_f32 (optional) its out_f32: the unrounded result is then read
    from there and the mixed row rounded once."""
    n_slots, n_kv_heads, n_sinks, head_dim = sink_k.shape
    _check_heads(n_heads, n_kv_heads, head_dim)
    T = q.shape[0]
    dt = q.dtype
    B = seq_slot.shape[0]
    if window < n_sinks:
        raise ValueError("a window of %d is narrower than the %d sinks beside it" % (window, n_sinks))
    n_pos, p_cs = 0, None
    if cos_sin is not None and rotary_dim > 0:
        n_pos = cos_sin.shape[0]
        p_cs = _need(cos_sin, "cos_sin", torch.float32, (n_pos, rotary_dim // 2, 2))
    library.check(library.lib().yalm_attn_sink_mix(
        _need(q, "q", dt, (T, n_heads * head_dim)), _need(out, "out", dt, (T, n_heads * head_dim)),
        _opt(src_f32, "src_f32", torch.float32, (T, n_heads * head_dim)),
        _need(lse, "lse", torch.float32, (T, n_heads)), _need(sink_k, "sink_k", dt),
        _need(sink_v, "sink_v", dt, (n_slots, n_kv_heads, n_sinks, head_dim)),
        _need(tok_seq, "tok_seq", torch.int32, (T,)), _need(tok_pos, "tok_pos", torch.int32, (T,)),
        _need(seq_slot, "seq_slot", torch.int32, (B,)), p_cs, n_pos, T, n_slots, n_heads, n_kv_heads, head_dim,
        int(rotary_dim) if p_cs is not None else 0, int(window), n_sinks, dtype_code(dt), _stream()), "attn_sink_mix")
    return out


# ---------------------------------------------------------------------------------------------------------------
# layers that norm a sublayer's output; PolyNorm
def cast(x, out):
    """out = x (float32) in out's dtype, element by element."""
    n = x.numel()
    if out.numel() != n:
        raise ValueError("cast: %d elements into %d" % (n, out.numel()))
    library.check(library.lib().yalm_cast(_need(x, "x", torch.float32), _need(out, "out"), n, dtype_code(out.dtype),
                                          _stream()), "cast")
    return out


def norm_add(y, weight, eps, x, h_out=None, next_norm=None):
    """x += y * rsqrt(mean(y^2) + eps) * weight, row by row (x, y float32 [R, D]); h_out (optional, [R, D] in the
    compute dtype) receives the new x: the input of the sublayer that follows; with next_norm = (float32 weights [D],
    eps) it receives the RMS norm of the new x with those weights instead (the norm that reads the stream next)."""
    R, D = y.shape
    p_h, h_code = None, 0
    if h_out is not None:
        p_h, h_code = _need(h_out, "h_out", None, (R, D)), dtype_code(h_out.dtype)
    p_n, n_eps = None, 0.0
    if next_norm is not None:
        if h_out is None:
            raise ValueError("norm_add: the next norm's output needs h_out")
        p_n, n_eps = _need(next_norm[0], "next norm weight", torch.float32, (D,)), float(next_norm[1])
    library.check(library.lib().yalm_norm_add(
        _need(y, "y", torch.float32, (R, D)), _need(weight, "weight", None, (D,)), dtype_code(weight.dtype), float(eps),
        _need(x, "x", torch.float32, (R, D)), p_h, h_code, p_n, n_eps, R, D, _stream()), "norm_add")
    return x


def polynorm(z, coef, eps, out):
    """out[r] = a N(z[r]) + b N(z[r]^2) + c N(z[r]^3) + e, powers element by element, N(v) = v / sqrt(mean(v^2) + eps);
    z float32 [R, F], coef float32 [4] = (a, b, c, e) on the device, out [R, F] in the compute dtype."""
    R, F = z.shape
    library.check(library.lib().yalm_polynorm(
        _need(z, "z", torch.float32, (R, F)), _need(coef, "coef", torch.float32, (4,)), float(eps),
        _need(out, "out", None, (R, F)), dtype_code(out.dtype), R, F, _stream()), "polynorm")
    return out


# ---------------------------------------------------------------------------------------------------------------
# latent attention
HEAD_MATMUL_MAX_K = 512


HEAD_MATMUL_MFMA_MIN_ROWS = 64


def head_matmul(src, src_head, src_off, wt, out, out_head, out_off, scale=1.0, gate=None, wt_nk=None):
    """For every row t and head h: out[t, h * out_head + out_off + n] = scale * sum_k src[t, h * src_head + src_off + k]
    * wt[h, k, n], times sigmoid(gate[t, h * N + n]) if gate (float32 [T, >= H * N]) is given.  src and out are
    2-D, their rows may be wider than the heads they hold; wt [H, K, N].  Types (src, wt, out): all float32;
    float32, bfloat16, float32; all bfloat16.  wt_nk (optional; bfloat16 [H, N, K], wt with its last axes exchanged): with
    HEAD_MATMUL_MFMA_MIN_ROWS rows or more, and sizes that keep 8 values of a row aligned, the product runs on the matrix
    cores (the rows rounded to bfloat16)."""
    H, K, N = wt.shape
    T = src.shape[0]
    mfma = (wt_nk is not None and T >= HEAD_MATMUL_MFMA_MIN_ROWS and not FORCE_SIMPLE and wt_nk.dtype == torch.bfloat16
            and K % 8 == 0 and src.shape[1] % 8 == 0 and src_head % 8 == 0 and src_off % 8 == 0)
    if K > HEAD_MATMUL_MAX_K:
        raise ValueError("head_matmul: %d inner elements a head, at most %d" % (K, HEAD_MATMUL_MAX_K))
    if src_off + K > src_head or out_off + N > out_head or H * src_head > src.shape[1] or H * out_head > out.shape[1]:
        raise ValueError("head_matmul: %d heads of %d (+%d) -> %d (+%d) do not fit rows of %d and %d"
                         % (H, K, src_off, N, out_off, src.shape[1], out.shape[1]))
    p_g, g_row = None, 0
    if gate is not None:
        g_row = gate.stride(0)
        if gate.dim() != 2 or gate.shape[0] != T or gate.shape[1] < H * N or gate.stride(1) != 1 \
                or gate.dtype != torch.float32 or not gate.is_cuda:
            raise ValueError("head_matmul: gate must be float32 [T, >= heads * N] with unit column stride on the GPU")
        p_g = gate.data_ptr()
    if mfma:
        library.check(library.lib().yalm_head_matmul_mfma(
            _need(src, "src", None, (T, None)), dtype_code(src.dtype), src.shape[1], src_head, src_off,
            _need(wt_nk, "wt_nk", torch.bfloat16, (H, N, K)), _need(out, "out", None, (T, None)), dtype_code(out.dtype),
            out.shape[1], out_head, out_off, float(scale), p_g, g_row, T, H, K, N, _stream()), "head_matmul on the matrix cores")
        return out
    library.check(library.lib().yalm_head_matmul(
        _need(src, "src", None, (T, None)), dtype_code(src.dtype), src.shape[1], src_head, src_off,
        _need(wt, "wt"), dtype_code(wt.dtype), _need(out, "out", None, (T, None)), dtype_code(out.dtype), out.shape[1],
        out_head, out_off, float(scale), p_g, g_row, T, H, K, N, _stream()), "head_matmul")
    return out


def latent_pack(proj, q_head, q_rot_off, kv_off, norm_w, eps, q_scale, out, n_heads, rot, rank, padded, has_kv):
    """Fills out float32 [T, (n_heads + 2) * padded], the rows that rope_kv_write reads as n_heads query heads and
    one KV head of size `padded`, each [rot | rank | zeros]: the rotated parts of the queries from proj (float32
    [T, *]; head h at column h * q_head + q_rot_off) times q_scale, zeros in the padding, and with has_kv the key
    [proj[kv_off + rank:][:rot] | c | 0] and the value [0 | c | 0], c the RMS norm (weights norm_w, eps) of
    proj[kv_off:][:rank].  The queries' rank places are left for head_matmul."""
    T = proj.shape[0]
    p_n, n_code = None, 0
    if has_kv:
        p_n, n_code = _need(norm_w, "norm_w", None, (rank,)), dtype_code(norm_w.dtype)
    library.check(library.lib().yalm_latent_pack(
        _need(proj, "proj", torch.float32, (T, None)), proj.shape[1], q_head, q_rot_off, kv_off if has_kv else 0, p_n,
        n_code, float(eps), float(q_scale), _need(out, "out", torch.float32, (T, (n_heads + 2) * padded)), T, n_heads,
        rot, rank, padded, 1 if has_kv else 0, _stream()), "latent_pack")
    return out


def can_v_tiles(pad, dtype):
    """Whether v_tiles takes heads of this width (a tile of 64 tokens of a head waits in 64 KB of LDS)."""
    return pad % 16 == 0 and PAGE * (pad + 8) * (4 if dtype == torch.float32 else 2) <= 64 * 1024


def v_tiles(v_rows, v_stage, v_pages, cu_seqlens, seq_tile0, block_table, ring_pages, seq_slot, seq_len, n_kv_heads, pad):
    """The values that qkv_pack left row by row (v_rows [T, G pad]) into the transposed staging tiles [n_tiles, G, pad,
    64] and cache pages (None: nowhere) of a step of whole prompts, a tile of 64 tokens at a time."""
    T = v_rows.shape[0]
    dt = v_rows.dtype
    B = seq_slot.shape[0]
    n_tiles = v_stage.shape[0]
    if not can_v_tiles(pad, dt):
        raise ValueError("v_tiles: heads of %d are too wide" % pad)
    n_pages, stride = 0, 0
    if v_pages is not None:
        n_pages, stride = v_pages.shape[0], block_table.shape[1]
        if ring_pages <= 0 or ring_pages > stride:
            raise ValueError("ring_pages %d does not fit the block table (%d columns)" % (ring_pages, stride))
    library.check(library.lib().yalm_v_tiles(
        _need(v_rows, "v_rows", dt, (T, n_kv_heads * pad)), _need(v_stage, "v_stage", dt, (n_tiles, n_kv_heads, pad, PAGE)),
        _opt(v_pages, "v_pages", dt, (n_pages, n_kv_heads, pad, PAGE)), _need(cu_seqlens, "cu_seqlens", torch.int32, (B + 1,)),
        _need(seq_tile0, "seq_tile0", torch.int32, (B + 1,)), _opt(block_table, "block_table", torch.int32, (None, None)), stride,
        int(ring_pages), _need(seq_slot, "seq_slot", torch.int32, (B,)), _opt(seq_len, "seq_len", torch.int32, (B,)), B, n_tiles,
        n_kv_heads, pad, n_pages, page_layout(pad), dtype_code(dt), _stream()), "v_tiles")
    return v_stage


def qkv_pack(qkv, bias, w_q, w_k, eps, q_temp, q_scale, v_first, blend, lam, q_out, k_stage, v_stage, seq_tile0, k_pages,
             v_pages, block_table, ring_pages, tok_seq, tok_pos, seq_slot, seq_len, n_heads, n_kv_heads, d, dv, pad,
             v_rows=None, head_norm=False, v_from_k=False, cos_sin=None, rot_dims=0):
    """From a q/k/v product to an attention without rotation.  qkv float32 [T, H d + G d + G dv] (+ bias, float32 of
    that width or None); RMS norms over the WHOLE query and key projections with the weights w_q [H d], w_k [G d]
    (float32; None: no norm); the queries times q_scale and, with q_temp = (coef, every), times 1 + coef ln(floor((p + 1)
    / every) + 1) at position p; blend 1 stores the values in v_first (float32 [T, G dv]), blend 2 replaces them by
    (1 - lam) v + lam v_first (lam: one float32 on the device).  Heads are written `pad` wide, zeros behind: q_out [T,
    H pad]; keys and values into the cache pages (None: nowhere) and, with k_stage, into the staging tiles of a step of
    whole prompts.  v_rows ([T, G pad], optional): the values go there row by row instead (v_tiles then transposes them).
    head_norm: the norms run over each head's d elements instead, w_q and w_k being [d] and shared by the heads.
    v_from_k: qkv is [T, H d + G d] only and a head's values are its keys as projected, before their norm (dv = d).
    rot_dims > 0 with cos_sin (float32 [positions, rot_dims / 2, 2]): behind the norms the neighbours (2p, 2p + 1) of
    every query and key head's first rot_dims elements are turned by the angle of pair p at the token's position."""
    T = qkv.shape[0]
    Q, K, V = n_heads * d, n_kv_heads * d, n_kv_heads * dv
    N = Q + K + (0 if v_from_k else V)
    if v_from_k and (d != dv or blend):
        raise ValueError("qkv_pack: values taken from the keys are as wide as the keys, and are not blended")
    rot_dims = int(rot_dims or 0)
    n_pos = 0
    if rot_dims:
        if rot_dims % 2 or rot_dims > d or cos_sin is None:
            raise ValueError("qkv_pack: %d turned elements do not fit heads of %d, or the table of angles is missing" % (rot_dims, d))
        n_pos = cos_sin.shape[0]
    dt = q_out.dtype
    if pad < max(d, dv) or N * 4 > 64 * 1024:
        raise ValueError("qkv_pack: heads of %d and %d do not fit %d, or a row of %d values is too wide" % (d, dv, pad, N))
    if blend not in (0, 1, 2) or (blend and v_first is None) or (blend == 2 and lam is None):
        raise ValueError("qkv_pack: blend %r needs v_first (and lam)" % (blend,))
    coef, every = q_temp if q_temp else (0.0, 0)
    n_pages = 0 if k_pages is None else k_pages.shape[0]
    n_tiles = 0 if k_stage is None else k_stage.shape[0]
    stride = 0
    if k_pages is not None:
        stride = block_table.shape[1]
        if ring_pages <= 0 or ring_pages > stride:
            raise ValueError("ring_pages %d does not fit the block table (%d columns)" % (ring_pages, stride))
    library.check(library.lib().yalm_qkv_pack(
        _need(qkv, "qkv", torch.float32, (T, N)), _opt(bias, "bias", torch.float32, (N,)),
        _opt(w_q, "w_q", torch.float32, (d if head_norm else Q,)), _opt(w_k, "w_k", torch.float32, (d if head_norm else K,)),
        float(eps), float(coef), int(every),
        float(q_scale), _opt(v_first, "v_first", torch.float32, (T, V)), int(blend), _opt(lam, "lam", torch.float32),
        _need(q_out, "q_out", dt, (T, n_heads * pad)),
        _opt(k_stage, "k_stage", dt, (n_tiles, n_kv_heads, PAGE, pad)),
        _opt(v_stage, "v_stage", dt, (n_tiles, n_kv_heads, pad, PAGE)),
        _opt(seq_tile0, "seq_tile0", torch.int32), _opt(k_pages, "k_pages", dt, (n_pages, n_kv_heads, PAGE, pad)),
        _opt(v_pages, "v_pages", dt, (n_pages, n_kv_heads, pad, PAGE)), _opt(block_table, "block_table", torch.int32, (None, None)),
        stride, int(ring_pages), _need(tok_seq, "tok_seq", torch.int32, (T,)), _need(tok_pos, "tok_pos", torch.int32, (T,)),
        _need(seq_slot, "seq_slot", torch.int32), _opt(seq_len, "seq_len", torch.int32), T, n_heads, n_kv_heads, d, dv, pad,
        n_pages, page_layout(pad), dtype_code(dt), _opt(v_rows, "v_rows", dt, (T, n_kv_heads * pad)),
        1 if head_norm else 0, 1 if v_from_k else 0,
        _need(cos_sin, "cos_sin", torch.float32, (n_pos, rot_dims // 2, 2)) if rot_dims else None, rot_dims, n_pos,
        _stream()), "qkv_pack")
    return q_out


MLSTM_MAX_VDIM = 256             # a thread of the recurrence's workgroup owns one column of the state
MLSTM_MAX_LDS = 150 * 1024


def mlstm_fits(d, dv):
    """Whether mlstm_scan takes heads of these sizes (the state of a head waits in LDS)."""
    groups = max(1, min(256 // max(dv, 1), d))
    return 0 < dv <= MLSTM_MAX_VDIM and d > 0 and (d * dv + 3 * d + dv + groups * dv) * 4 <= MLSTM_MAX_LDS


def mlstm_chunk(d, prompt):
    """The chunk with which mlstm_chunks takes key heads of d: 64 tokens for steps of whole prompts where that fits its
    LDS, else 16; 0 if not even that fits (mlstm_scan then serves)."""
    for chunk in ((64, 16) if prompt else (16,)):
        if library.lib().yalm_mlstm_chunks_lds(int(d), chunk) <= MLSTM_MAX_LDS:
            return chunk
    return 0


def mlstm_chunks(proj, b_i, b_f, w_norm, state, raw, nm, cu_seqlens, seq_slot, out, n_heads, d, dv, q_scale, cap, floor, eps,
                 chunk):
    """mlstm_scan's result a chunk of `chunk` tokens at a time on the matrix cores, in float32 arithmetic (the same
    recurrence written over a chunk: scores q . k weighted by the gates inside it, the state carried between chunks).
    raw float32 [T, H dv] and nm float32 [B, H (d + 1)] are scratch."""
    T = proj.shape[0]
    B = seq_slot.shape[0]
    H = n_heads
    if chunk not in (16, 64) or library.lib().yalm_mlstm_chunks_lds(int(d), chunk) > MLSTM_MAX_LDS:
        raise ValueError("mlstm_chunks: key heads of %d do not fit chunks of %r" % (d, chunk))
    n_slots = state.shape[0]
    library.check(library.lib().yalm_mlstm_chunks(
        _need(proj, "proj", torch.float32, (T, 2 * H * d + 2 * H * dv + 2 * H)), _need(b_i, "b_i", torch.float32, (H,)),
        _need(b_f, "b_f", torch.float32, (H,)), _need(w_norm, "w_norm", torch.float32, (H * dv,)),
        _need(state, "state", torch.float32, (n_slots, H * (d * dv + d + 1))), _need(raw, "raw", torch.float32, (T, H * dv)),
        _need(nm, "nm", torch.float32, (B, H * (d + 1))), _need(cu_seqlens, "cu_seqlens", torch.int32, (B + 1,)),
        _need(seq_slot, "seq_slot", torch.int32, (B,)), _need(out, "out", None, (T, H * dv)), T, B, H, d, dv, float(q_scale),
        float(cap), float(floor), float(eps), n_slots, int(chunk), dtype_code(out.dtype), _stream()), "mlstm_chunks")
    return out


def mlstm_scan(proj, b_i, b_f, w_norm, state, cu_seqlens, seq_slot, out, n_heads, d, dv, q_scale, cap, floor, eps):
    """The matrix-memory recurrence over the tokens of a step.  proj float32 [T, 2 H d + 2 H dv + 2 H] = q | k | v | g |
    z_i | z_f; with i = cap tanh((z_i + b_i) / cap), f = logsigmoid(cap tanh((z_f + b_f) / cap)) (cap 0: uncapped):
    m' = max(f + m, i), S' = exp(f + m - m') S + exp(i - m') k v^T, n' likewise with k, o = S'^T (q q_scale) / (max(|n' .
    q|, exp(-m')) + floor); out [T, H dv] = o / rms(o) (a head at a time) * w_norm * sigmoid(g).  state float32
    [slots, H (d dv + d + 1)] is read and left advanced; the tokens of sequence b are the rows cu_seqlens[b] ..
    cu_seqlens[b + 1] - 1, in order; rows with seq_slot < 0 are left alone."""
    T = proj.shape[0]
    B = seq_slot.shape[0]
    H = n_heads
    if not mlstm_fits(d, dv):
        raise ValueError("mlstm_scan: heads of %d x %d are not offered" % (d, dv))
    n_slots = state.shape[0]
    library.check(library.lib().yalm_mlstm_scan(
        _need(proj, "proj", torch.float32, (T, 2 * H * d + 2 * H * dv + 2 * H)), _need(b_i, "b_i", torch.float32, (H,)),
        _need(b_f, "b_f", torch.float32, (H,)), _need(w_norm, "w_norm", torch.float32, (H * dv,)),
        _need(state, "state", torch.float32, (n_slots, H * (d * dv + d + 1))),
        _need(cu_seqlens, "cu_seqlens", torch.int32, (B + 1,)), _need(seq_slot, "seq_slot", torch.int32, (B,)),
        _need(out, "out", None, (T, H * dv)), B, H, d, dv, float(q_scale), float(cap), float(floor), float(eps), n_slots,
        dtype_code(out.dtype), _stream()), "mlstm_scan")
    return out


GATED_DELTA_MAX_KEY_DIM = 256     # a lane of the recurrence holds one column of a head's state in registers
GATED_DELTA_MAX_TAPS = 16


def gated_delta_state_elements(n_heads, n_qk_heads, d, dv, taps):
    """Floats of per-sequence state that gated_delta keeps: the heads' matrices and the convolutions' last inputs."""
    return n_heads * d * dv + (2 * n_qk_heads * d + n_heads * dv) * (taps - 1)


def gated_delta(proj, low, conv_w, decay_log, decay_bias, w_norm, state, prep, raw, tok_seq, cu_seqlens, seq_slot, out,
                n_heads, n_qk_heads, d, dv, taps, q_scale, unit_floor, eps):
    """The gated delta rule with a decay per key channel over the tokens of a step, in float32.  proj float32
    [T, 2 Hq d + H dv + H] = q | k | v | b (before the short causal convolutions conv_w [2 Hq d + H dv, taps], whose last column
    is the current token's); low float32 [T, H d + H dv], the decay's and the output gate's pre-activations.  Per token:
    q, k, v <- silu(convolution); q, k unit vectors a head (x / sqrt(sum x^2 + unit_floor)), q times q_scale; beta =
    sigmoid(b); g = exp(-exp(decay_log[h]) softplus(low + decay_bias)); per head S <- diag(g) S, u = beta (v - S^T k),
    S <- S + k u^T, o = S^T q; out [T, H dv] = o / rms(o) (a head at a time) * w_norm [dv] * sigmoid(gate pre-activation).
    state float32 [slots, gated_delta_state_elements(...)] is read and left advanced; prep [T, 2 Hq d + H dv + H + H d] and raw
    [T, H dv] are float32 scratch.  The tokens of sequence b are the rows cu_seqlens[b] .. cu_seqlens[b + 1] - 1; rows of
    sequences with seq_slot < 0 are left alone."""
    T = proj.shape[0]
    B = seq_slot.shape[0]
    H, Hq = n_heads, n_qk_heads
    if not (0 < d <= GATED_DELTA_MAX_KEY_DIM and 0 < taps <= GATED_DELTA_MAX_TAPS and Hq > 0 and H % Hq == 0):
        raise ValueError("gated_delta: key heads of %d, %d taps, %d heads on %d query heads are not offered" % (d, taps, H, Hq))
    C = 2 * Hq * d + H * dv
    if 2 * Hq + (H * dv + 255) // 256 + (H * d + 255) // 256 > 65535:
        raise ValueError("gated_delta: %d heads of %d x %d are more than a launch's grid holds" % (H, d, dv))
    n_slots = state.shape[0]
    library.check(library.lib().yalm_gated_delta(
        _need(proj, "proj", torch.float32, (T, C + H)), _need(low, "low", torch.float32, (T, H * d + H * dv)),
        _need(conv_w, "conv_w", torch.float32, (C, taps)), _need(decay_log, "decay_log", torch.float32, (H,)),
        _need(decay_bias, "decay_bias", torch.float32, (H * d,)), _need(w_norm, "w_norm", torch.float32, (dv,)),
        _need(state, "state", torch.float32, (n_slots, gated_delta_state_elements(H, Hq, d, dv, taps))),
        _need(prep, "prep", torch.float32, (T, C + H + H * d)), _need(raw, "raw", torch.float32, (T, H * dv)),
        _need(tok_seq, "tok_seq", torch.int32, (T,)), _need(cu_seqlens, "cu_seqlens", torch.int32, (B + 1,)),
        _need(seq_slot, "seq_slot", torch.int32, (B,)), _need(out, "out", None, (T, H * dv)), T, B, H, Hq, d, dv, taps,
        float(q_scale), float(unit_floor), float(eps), n_slots, dtype_code(out.dtype), _stream()), "gated_delta")
    return out


def embed_learned(table, pos_table, tokens, positions, scale, out):
    """out[t] = table[tokens[t]] * scale + pos_table[positions[t]] (float32 out; both tables of one dtype)."""
    T = tokens.shape[0]
    V, D = table.shape
    P = pos_table.shape[0]
    library.check(library.lib().yalm_embed_learned(
        _need(table, "table", None, (V, D)), _need(pos_table, "pos_table", table.dtype, (P, D)), dtype_code(table.dtype),
        _need(tokens, "tokens", torch.int32, (T,)), _need(positions, "positions", torch.int32, (T,)), float(scale),
        _need(out, "out", torch.float32, (T, D)), T, D, V, P, _stream()), "embed_learned")
    return out


ACTIVATIONS = {"gelu_erf": 0, "gelu_tanh": 1, "silu": 2}


def activate(z, out, kind):
    """out = act(z), z float32, out of its own dtype and z's shape; kind: "gelu_erf" (z/2 (1 + erf(z / sqrt 2))),
    "gelu_tanh" or "silu"."""
    if kind not in ACTIVATIONS:
        raise ValueError("activation %r is not offered (%s)" % (kind, ", ".join(ACTIVATIONS)))
    library.check(library.lib().yalm_activate(_need(z, "z", torch.float32), _need(out, "out", None, tuple(z.shape)), z.numel(),
                                              ACTIVATIONS[kind], dtype_code(out.dtype), _stream()), "activate")
    return out


def gated_add(y, h, w, x, accumulate=True):
    """x[t] (+)= sigmoid(h[t] . w) * y[t]: a sublayer's result y (float32 [T, D]) under a gate of one number a token."""
    T, D = y.shape
    library.check(library.lib().yalm_gated_add(
        _need(y, "y", torch.float32, (T, D)), _need(h, "h", None, (T, D)), _need(w, "w", h.dtype, (D,)), dtype_code(h.dtype),
        _need(x, "x", torch.float32, (T, D)), T, D, 1 if accumulate else 0, _stream()), "gated_add")
    return x


TIME_CONV_MAX_TAPS = 16


def time_conv(h, w, carried, out, tok_seq, cu_seqlens, seq_slot, residual=True, one_token_each=False):
    """out[t, c] = (h[t, c] if residual) + sum_j w[j, c] in(t - (taps - 1) + j, c): a causal convolution over the tokens
    of each sequence of the step, the last tap on the token itself (h, out [T, D] of one dtype and not the same
    memory; w float32 [taps, D], tap by tap).  carried (float32 [slots, taps - 1, D]; None with one tap) holds each sequence's last
    taps - 1 inputs, read for the places in front of the step's first token and left advanced.  one_token_each: the caller
    knows that every sequence brings one token (row t is sequence t), which saves a launch."""
    T, D = h.shape
    taps = w.shape[0]
    B = seq_slot.shape[0]
    if not 0 < taps <= TIME_CONV_MAX_TAPS:
        raise ValueError("time_conv: %d taps (at most %d)" % (taps, TIME_CONV_MAX_TAPS))
    if h.data_ptr() == out.data_ptr():
        raise ValueError("time_conv: the result needs memory of its own")
    p_c = None
    if taps > 1:
        p_c = _need(carried, "carried", torch.float32, (None, taps - 1, D))
    library.check(library.lib().yalm_time_conv(
        _need(h, "h", None, (T, D)), _need(w, "w", torch.float32, (taps, D)), p_c, _need(out, "out", h.dtype, (T, D)),
        _need(tok_seq, "tok_seq", torch.int32, (T,)), _need(cu_seqlens, "cu_seqlens", torch.int32, (B + 1,)),
        _need(seq_slot, "seq_slot", torch.int32, (B,)), T, B, D, taps, 1 if residual else 0,
        1 if one_token_each and T == B else 0, dtype_code(h.dtype), _stream()),
        "time_conv")
    return out


def gated_bias_act(z, bias, out, kind, x=None, x_bias=None):
    """out[t, i] = act(z[t, i] + bias[i]) * (z[t, F + i] + bias[F + i]): z float32 [T, 2 F] (gate | up), bias float32
    [2 F] or None, out [T, F] of its own dtype; kind as in activate.  With x (float32 [T, D]) and x_bias (float32 [D])
    also x[t] += x_bias."""
    if kind not in ACTIVATIONS:
        raise ValueError("activation %r is not offered (%s)" % (kind, ", ".join(ACTIVATIONS)))
    T, F2 = z.shape
    F = F2 // 2
    D = 0
    p_x = p_xb = None
    if x_bias is not None:
        D = x.shape[1]
        p_x, p_xb = _need(x, "x", torch.float32, (T, D)), _need(x_bias, "x_bias", torch.float32, (D,))
    library.check(library.lib().yalm_gated_bias_act(
        _need(z, "z", torch.float32, (T, 2 * F)), _opt(bias, "bias", torch.float32, (2 * F,)), _need(out, "out", None, (T, F)),
        T, F, ACTIVATIONS[kind], dtype_code(out.dtype), p_x, p_xb, D, _stream()), "gated_bias_act")
    return out


def sigmoid_gate(o, g, n_heads, dv, pad):
    """o[t, h, e] *= sigmoid(g[t, h dv + e]) for e < dv: o [T, n_heads pad] in its own dtype, g float32 rows of a wider
    float32 matrix (a view whose rows are g.stride(0) apart)."""
    T = o.shape[0]
    if g.dtype != torch.float32 or g.dim() != 2 or g.shape != (T, n_heads * dv) or g.stride(1) != 1 or not g.is_cuda:
        raise ValueError("sigmoid_gate: the gates are float32 [%d, %d] on the device, rows contiguous" % (T, n_heads * dv))
    library.check(library.lib().yalm_sigmoid_gate(
        _need(o, "o", None, (T, n_heads * pad)), g.data_ptr(), int(g.stride(0)), T, n_heads, dv, pad, dtype_code(o.dtype),
        _stream()), "sigmoid_gate")
    return o


def loop_pack(x, x0, start, both):
    """both[t] = [x[t] | x0[t]] in both's dtype, then x[t] = start (x, x0 float32 [T, D]; start float32 [D])."""
    T, D = x.shape
    library.check(library.lib().yalm_loop_pack(
        _need(x, "x", torch.float32, (T, D)), _need(x0, "x0", torch.float32, (T, D)), _need(start, "start", torch.float32, (D,)),
        _need(both, "both", None, (T, 2 * D)), T, D, dtype_code(both.dtype), _stream()), "loop_pack")
    return both


HGRN2_MAX_KEY_DIM = 256           # a lane of the recurrence holds 32 rows of a state column at most


def hgrn2_state_elements(n_heads, d, dv):
    return n_heads * d * dv


def hgrn2(proj, f_bias, lower, w_norm, state, raw, cu_seqlens, seq_slot, out, n_heads, d, dv, eps):
    """The HGRN2 recurrence over a step's tokens.  proj float32 [T, 2 H d + H dv] = z_q | z_f | v; q = silu(z_q), f = lower
    + (1 - lower) sigmoid(z_f + f_bias); per head S <- diag(f) S + (1 - f) v^T, o = S^T q; out [T, H dv] = o over its root
    mean square a head, times w_norm [dv].  state float32 [slots, H dv d] (a head's S column by column) is read and left
    advanced; raw float32 [T, H dv] is scratch.  Sequence b's tokens are cu_seqlens[b] .. cu_seqlens[b + 1] - 1."""
    T = proj.shape[0]
    B = seq_slot.shape[0]
    N = 2 * n_heads * d + n_heads * dv
    if not 0 < d <= HGRN2_MAX_KEY_DIM:
        raise ValueError("hgrn2: key heads of %d (at most %d)" % (d, HGRN2_MAX_KEY_DIM))
    library.check(library.lib().yalm_hgrn2(
        _need(proj, "proj", torch.float32, (T, N)), _need(f_bias, "f_bias", torch.float32, (n_heads * d,)),
        _need(lower, "lower", torch.float32, (n_heads * d,)), _need(w_norm, "w_norm", torch.float32, (dv,)),
        _need(state, "state", torch.float32, (None, n_heads * d * dv)), _need(raw, "raw", torch.float32, (T, n_heads * dv)),
        _need(cu_seqlens, "cu_seqlens", torch.int32, (B + 1,)), _need(seq_slot, "seq_slot", torch.int32, (B,)),
        _need(out, "out", None, (T, n_heads * dv)), T, B, n_heads, d, dv, float(eps), dtype_code(out.dtype), _stream()), "hgrn2")
    return out


# ---------------------------------------------------------------------------------------------------------------
# mixture of experts
MOE_MAX_EXPERTS = 1024


def moe_route(h, w_router, ids, wts, renormalize=False):
    """ids, wts [T, top]: the top experts of every row of h [T, D] by softmax(w_router h) over all experts
    (float32 arithmetic, the lowest index on ties) and those scores (renormalize: divided by their sum)."""
    T, D = h.shape
    E = w_router.shape[0]
    top = ids.shape[1]
    if not 0 < top <= E or E > MOE_MAX_EXPERTS:
        raise ValueError("moe_route: %d of %d experts is not offered (at most %d experts)" % (top, E, MOE_MAX_EXPERTS))
    library.check(library.lib().yalm_moe_route(
        _need(h, "h", None, (T, D)), _need(w_router, "w_router", h.dtype, (E, D)), dtype_code(h.dtype),
        _need(ids, "ids", torch.int32, (T, top)), _need(wts, "wts", torch.float32, (T, top)), T, D, E, top,
        1 if renormalize else 0, _stream()), "moe_route")


def moe_select(logits, ids, wts, renormalize=False, bias=None):
    """moe_route from logits that a product has made already (float32 [T, E]); bias (float32 [E]) is added to them
    first.  renormalize "chosen": the experts with the largest logits, weighted by the softmax over the chosen logits
    alone (no score over all experts is formed)."""
    T, E = logits.shape
    top = ids.shape[1]
    if not 0 < top <= E or E > MOE_MAX_EXPERTS:
        raise ValueError("moe_select: %d of %d experts is not offered (at most %d experts)" % (top, E, MOE_MAX_EXPERTS))
    mode = 2 if renormalize == "chosen" else (1 if renormalize else 0)
    library.check(library.lib().yalm_moe_select(
        _need(logits, "logits", torch.float32, (T, E)), _opt(bias, "bias", torch.float32, (E,)),
        _need(ids, "ids", torch.int32, (T, top)), _need(wts, "wts", torch.float32, (T, top)), T, E, top, mode, _stream()),
        "moe_select")


def moe_pair_gate_up(h, w_gate, w_up, ids, limit, alpha, mid, up_shift=1.0):
    """mid[t * top + k] = g sigmoid(alpha g) (u + up_shift), g = min(w_gate[e] h[t], limit), u = clamp(w_up[e] h[t], +-limit)
    for e = ids[t, k] (limit <= 0: unclamped; alpha 1, up_shift 0: silu(gate) * up); w_gate, w_up [E, F, D]."""
    T, D = h.shape
    E, F, _ = w_gate.shape
    top = ids.shape[1]
    dt = h.dtype
    library.check(library.lib().yalm_moe_pair_gate_up(
        _need(h, "h", dt, (T, D)), _need(w_gate, "w_gate", dt, (E, F, D)), _need(w_up, "w_up", dt, (E, F, D)),
        _need(ids, "ids", torch.int32, (T, top)), float(limit), float(alpha), float(up_shift),
        _need(mid, "mid", dt, (T * top, F)), T, top, D, F, E, dtype_code(dt), _stream()), "moe_pair_gate_up")
    return mid


def moe_pair_down(mid, w_down, ids, wts, out, accumulate=False):
    """out float32 [T, D] = (accumulate: out +) sum over k, in order, of wts[t, k] * w_down[ids[t, k]] mid[t * top + k]; w_down [E, D, F]."""
    E, D, F = w_down.shape
    T, top = ids.shape
    dt = mid.dtype
    library.check(library.lib().yalm_moe_pair_down(
        _need(mid, "mid", dt, (T * top, F)), _need(w_down, "w_down", dt, (E, D, F)),
        _need(ids, "ids", torch.int32, (T, top)), _need(wts, "wts", torch.float32, (T, top)),
        _need(out, "out", torch.float32, (T, D)), T, top, D, F, E, dtype_code(dt), 1 if accumulate else 0, _stream()), "moe_pair_down")
    return out



MOE_GROUP_ROWS = 128           # rows of a tile of the grouped products (csrc/moe.hip)


def can_moe_grouped(D, F, dtype, n_pairs=0, n_experts=0):
    """Whether moe_grouped takes these sizes (and this many pairs: its tiles are one axis of a launch)."""
    return dtype == torch.bfloat16 and D % 8 == 0 and F % 8 == 0 and not FORCE_SIMPLE \
        and (n_pairs + MOE_GROUP_ROWS - 1) // MOE_GROUP_ROWS + n_experts <= 65535


def moe_grouped_tiles(n_pairs, n_experts):
    """Tiles of MOE_GROUP_ROWS rows that the grouped products need at most for n_pairs (token, choice) pairs."""
    return library.lib().yalm_moe_grouped_tiles(int(n_pairs), int(n_experts))


def moe_grouped(h, w_gate, w_up, w_down, ids, wts, limit, alpha, scratch, out, accumulate=False, up_shift=1.0):
    """What moe_pair_gate_up + moe_pair_down compute, for many tokens (bfloat16): the pairs are grouped by expert on
    the device and every product is one launch over all experts' tiles on the matrix cores.  scratch(name, shape,
    dtype) hands out the buffers (pair_of_row, row_of_pair, tile_expert, mid, y)."""
    T, D = h.shape
    E, F, _ = w_gate.shape
    top = ids.shape[1]
    dt = torch.bfloat16
    tiles = moe_grouped_tiles(T * top, E)
    rows = tiles * MOE_GROUP_ROWS
    pair_of_row = scratch("moe.pair_of_row", (rows,), torch.int32)
    row_of_pair = scratch("moe.row_of_pair", (T * top,), torch.int32)
    tile_expert = scratch("moe.tile_expert", (tiles,), torch.int32)
    mid = scratch("moe.hidden", (rows, F), dt)
    y = scratch("moe.y", (rows, D), torch.float32)
    library.check(library.lib().yalm_moe_grouped(
        _need(h, "h", dt, (T, D)), _need(w_gate, "w_gate", dt, (E, F, D)), _need(w_up, "w_up", dt, (E, F, D)),
        _need(w_down, "w_down", dt, (E, D, F)), _need(ids, "ids", torch.int32, (T, top)),
        _need(wts, "wts", torch.float32, (T, top)), float(limit), float(alpha), float(up_shift),
        _need(pair_of_row, "pair_of_row", torch.int32, (rows,)), _need(row_of_pair, "row_of_pair", torch.int32, (T * top,)),
        _need(tile_expert, "tile_expert", torch.int32, (tiles,)), _need(mid, "mid", dt, (rows, F)),
        _need(y, "y", torch.float32, (rows, D)), _need(out, "out", torch.float32, (T, D)), T, top, D, F, E,
        1 if accumulate else 0, _stream()), "moe_grouped")
    return out


def argmax(logits, out):
    R, V = logits.shape
    library.check(library.lib().yalm_argmax(_need(logits, "logits", torch.float32), _need(out, "out", torch.int32, (R,)),
                                            R, V, _stream()), "argmax")
    return out


def sample(logits, u, temperature, out):
    R, V = logits.shape
    if not temperature > 0:
        raise ValueError("temperature must be positive here (0 is argmax)")
    library.check(library.lib().yalm_sample(_need(logits, "logits", torch.float32), _need(u, "u", torch.float32, (R,)),
                                            float(temperature), _need(out, "out", torch.int32, (R,)), R, V, _stream()),
                  "sample")
    return out


def token_prob(logits, index, out):
    R, V = logits.shape
    library.check(library.lib().yalm_token_prob(_need(logits, "logits", torch.float32),
                                                _need(index, "index", torch.int32, (R,)),
                                                _need(out, "out", torch.float32, (R,)), R, V, _stream()), "token_prob")
    return out


def probe_read(src, workgroups=2048):
    """Queues a kernel that reads the tensor `src` once and does nothing else (a yardstick for what the
    memory gives a kernel).  Returns the bytes it reads."""
    n = src.numel() * src.element_size()
    piece = 256 * 8 * 16
    if n < piece:
        raise ValueError("probe_read needs at least %d bytes" % piece)
    out = _probe_scratch(src.device)
    library.check(library.lib().yalm_probe_read(_need(src, "src"), n, out.data_ptr(), int(workgroups), _stream()),
                  "probe_read")
    return n // piece * piece


def probe_mfma(shape, iters, workgroups=2048):
    """Queues a loop of matrix-core instructions on registers (shape 32: 32x32x16, 16: 16x16x32, bfloat16).
    Returns the floating-point operations of the launch."""
    out = _probe_scratch(torch.device("cuda", torch.cuda.current_device()))
    flops = ctypes.c_double(0.0)
    library.check(library.lib().yalm_probe_mfma(int(shape), int(iters), int(workgroups), out.data_ptr(),
                                                ctypes.byref(flops), _stream()), "probe_mfma")
    return flops.value


_probe_out = {}


def _probe_scratch(device):
    key = str(device)
    if key not in _probe_out:
        _probe_out[key] = torch.zeros(1024, dtype=torch.int32, device=device)
    return _probe_out[key]
