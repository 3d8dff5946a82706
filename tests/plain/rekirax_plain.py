"""A plain, slow implementation of the Rekirax design in float64 torch on the CPU: one function per
mechanism, written from the design's equations and sharing nothing with yalm_amd.  The tests hold the
library against it.

The design: a decoder whose token embedding is normed at once; whose layers are pre-norm
(x <- x + mixer(c(n1(x))); x <- x + ff(n2(x)), the norms' weights stored as their distance from one, c a short
causal convolution over time added to its own input); a run of layers may be walked several times with the same
weights, every walk with memories of its own, entered through a matrix on [x; embedding output] and a vector of
the walk.  The mixers: a grouped-query attention under a sliding window whose values are its un-normed keys, with
norms a head, capped scores and a term that grows with the logarithm of the distance; or two mixers side by
side, a rotary attention inside chunks of positions with norms over whole projections and an output gate, and a
gated linear recurrence whose forget gate also decides what is written (HGRN2), each normed over the width and
the two averaged.  Feed-forwards are gated with the tanh gelu and carry biases.  The head is the embedding table.

`weights` is a dictionary name -> tensor with the names of a model folder ('l3.mix.left.q', ...).  `memory`,
where a function takes one, is what a layer keeps of earlier tokens of ONE sequence: a dictionary the
functions fill and read, so that a text can be fed in pieces."""
import math

import torch

F64 = torch.float64


def W(w, name):
    return w[name].to(F64)


def rms_div(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_one_plus(x, w_around_zero, eps):
    """The layers' norm: the stored weight is the distance from one."""
    return rms_div(x, eps) * (1.0 + w_around_zero)


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ------------------------------------------------------------------------------------------ embedding, loop
def embed(tokens, w, eps):
    return norm_one_plus(W(w, "embed")[torch.tensor(tokens, dtype=torch.long)], W(w, "embed.norm"), eps)


def loop_entry(x, x0, w, t):
    """What a walk of the looped layers starts from: a matrix on [x; x0] (x first), plus the walk's vector."""
    return torch.cat([x, x0], dim=-1) @ W(w, "loop.in").T + W(w, "loop.step")[t]


def run_order(n_layers, loop):
    """[(layer, walk)] in the order in which layers run: the layers start..stop-1 `times` times in a row."""
    if not loop:
        return [(i, 0) for i in range(n_layers)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, 0) for i in range(start)]
    for t in range(times):
        order += [(i, t) for i in range(start, stop)]
    return order + [(i, 0) for i in range(stop, n_layers)]


# ------------------------------------------------------------------------------------------ input convolution
def input_conv(h, taps_w, memory):
    """h + conv(h): conv(h)[t, c] = sum_j taps_w[c, j] h[t - (n - 1) + j, c] with n taps, the last tap on the token
    itself, zeros before the sequence's start; the last n - 1 inputs wait in memory['conv']."""
    n = taps_w.shape[1]
    before = memory.get("conv")
    if before is None:
        before = torch.zeros((n - 1, h.shape[1]), dtype=F64)
    full = torch.cat([before, h])
    y = h.clone()
    for j in range(n):
        y = y + taps_w[:, j] * full[j:j + h.shape[0]]
    memory["conv"] = full[full.shape[0] - (n - 1):]
    return y


# ------------------------------------------------------------------------------------------ attentions
def sees_window(i, j, size):
    """Whether the query at i sees the key at j under a sliding window of `size` positions (itself included)."""
    return 0 <= i - j < size


def sees_chunk(i, j, size):
    """Whether the query at i sees the key at j when positions are cut into chunks of `size` from position 0."""
    return j <= i and i // size == j // size


def rotate_half(x, positions, dims, base):
    """x [T, heads, d]: of each head's first `dims` elements, element i and element i + dims/2 are turned by the
    angle position * base^(-2i/dims); the other elements pass."""
    if not dims:
        return x
    half = dims // 2
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = torch.tensor(positions, dtype=F64)[:, None, None] * f
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * torch.cos(a) - v * torch.sin(a), v * torch.cos(a) + u * torch.sin(a), x[..., dims:]], dim=-1)


def softmax_over_visible(q, keys, values, positions, scale, sees, shape_score=None):
    """q [T, H, d] at `positions`, keys [S, G, d] and values [S, G, dv] from position 0 on.  For every query and head
    the softmax over the keys that `sees(i, j)` lets through of scale * q . k, passed through shape_score(score,
    head, distance) if given.  Returns [T, H, dv]."""
    T, H, _ = q.shape
    S, G, dv = values.shape
    out = torch.zeros((T, H, dv), dtype=F64)
    for t, p in enumerate(positions):
        idx = torch.tensor([j for j in range(S) if sees(p, j)], dtype=torch.long)
        dist = p - idx.to(F64)
        for hd in range(H):
            g = hd // (H // G)
            s = (keys[idx, g] @ q[t, hd]) * scale
            if shape_score is not None:
                s = shape_score(s, hd, dist)
            out[t, hd] = torch.softmax(s, dim=0) @ values[idx, g]
    return out


def remember(memory, k, v):
    keys = torch.cat([memory["k"], k]) if "k" in memory else k
    values = torch.cat([memory["v"], v]) if "v" in memory else v
    memory["k"], memory["v"] = keys, values
    return keys, values


def window_projections(h, mixer, w, prefix, eps):
    """(q [T, H, d] and k [T, G, d], each head normed with a weight of d elements that the heads share; the keys as
    projected [T, G, d], which are the values)."""
    H, G, d = int(mixer["heads"]), int(mixer["kv_heads"]), int(mixer["dim"])
    T = h.shape[0]
    q = (h @ W(w, prefix + "q").T).reshape(T, H, d)
    k_raw = (h @ W(w, prefix + "k").T).reshape(T, G, d)
    return rms_div(q, eps) * W(w, prefix + "q.norm"), rms_div(k_raw, eps) * W(w, prefix + "k.norm"), k_raw


def chunk_projections(h, positions, mixer, w, prefix, eps):
    """(q [T, H, d], k [T, G, d], v [T, G, dv]): norms over the whole query and key projections, then the rotation."""
    H, G, d, dv = int(mixer["heads"]), int(mixer["kv_heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = rms_div(h @ W(w, prefix + "q").T, eps) * W(w, prefix + "q.norm")
    k = rms_div(h @ W(w, prefix + "k").T, eps) * W(w, prefix + "k.norm")
    v = (h @ W(w, prefix + "v").T).reshape(T, G, dv)
    rot = mixer.get("rot") or {}
    dims, base = int(rot.get("dims", 0) or 0), float(rot.get("base", 10000.0))
    return rotate_half(q.reshape(T, H, d), positions, dims, base), rotate_half(k.reshape(T, G, d), positions, dims, base), v


def window_attention(h, positions, mixer, w, prefix, eps, memory):
    """The mixer 'attention': keys double as values (as projected, before their norm); norms a head; capped scores
    less r1 ln(1 + r2 distance); a sliding window."""
    H, d = int(mixer["heads"]), int(mixer["dim"])
    T = h.shape[0]
    q, k, k_raw = window_projections(h, mixer, w, prefix, eps)
    keys, values = remember(memory, k, k_raw)
    assert keys.shape[0] == positions[-1] + 1
    cap = float(mixer.get("softcap") or 0.0)
    r1, r2 = W(w, prefix + "r1"), W(w, prefix + "r2")
    size = int(mixer["mask"]["size"]) if mixer.get("mask") else 1 << 60

    def shape_score(s, hd, dist):
        if cap:
            s = cap * torch.tanh(s / cap)
        return s - r1[hd] * torch.log(1.0 + r2[hd] * dist)

    o = softmax_over_visible(q, keys, values, positions, float(mixer["scale"]), lambda i, j: sees_window(i, j, size), shape_score)
    return o.reshape(T, H * d) @ W(w, prefix + "o").T


def chunk_attention(h, positions, mixer, w, prefix, eps, memory):
    """The left half of the mixer 'parallel': norms over the whole projections, then rotation of the heads' first
    elements; chunks of positions; the heads times sigmoid(W_g h) before the output projection."""
    H, dv = int(mixer["heads"]), int(mixer["vdim"])
    T = h.shape[0]
    q, k, v = chunk_projections(h, positions, mixer, w, prefix, eps)
    keys, values = remember(memory, k, v)
    assert keys.shape[0] == positions[-1] + 1
    size = int(mixer["mask"]["size"]) if mixer.get("mask") else 1 << 60
    o = softmax_over_visible(q, keys, values, positions, float(mixer["scale"]), lambda i, j: sees_chunk(i, j, size))
    gate = torch.sigmoid(h @ W(w, prefix + "g").T)
    return (o.reshape(T, H * dv) * gate) @ W(w, prefix + "o").T


# ------------------------------------------------------------------------------------------ HGRN2
def forget_gates(h, w, prefix):
    """f = l + (1 - l) sigmoid(W_f h + b): never under the lower bound l."""
    low = W(w, prefix + "lower")
    return low + (1.0 - low) * torch.sigmoid(h @ W(w, prefix + "f").T + W(w, prefix + "f.b"))


def hgrn2_recurrence(q, f, v, S):
    """q, f [T, H, d], v [T, H, dv], S [H, d, dv] -> (o [T, H, dv], S): S <- diag(f) S + (1 - f) v^T; o = S^T q."""
    T, H, dv = v.shape
    o = torch.zeros((T, H, dv), dtype=F64)
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return o, S


def hgrn2(h, mixer, w, prefix, eps, memory, reads_out=None):
    """reads_out, if a list, receives [T]: the smallest root mean square among the heads' results before their norm,
    which divides by it (a head that reads next to nothing from its state is normed up from rounding's leavings)."""
    H, d, dv = int(mixer["heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = silu(h @ W(w, prefix + "q").T).reshape(T, H, d)
    f = forget_gates(h, w, prefix).reshape(T, H, d)
    v = (h @ W(w, prefix + "v").T).reshape(T, H, dv)
    S = memory.get("S")
    if S is None:
        S = torch.zeros((H, d, dv), dtype=F64)
    o, memory["S"] = hgrn2_recurrence(q, f, v, S)
    if reads_out is not None:
        reads_out.append(torch.sqrt((o * o).mean(dim=-1)).min(dim=-1).values)
    o = rms_div(o, eps) * W(w, prefix + "norm")
    return o.reshape(T, H * dv) @ W(w, prefix + "o").T


def parallel_mixer(h, positions, mixer, w, prefix, eps, memory, reads_out=None):
    """Half the sum of the two mixers' results, each normed over the width with a plain weight of its own."""
    left = chunk_attention(h, positions, mixer["left"], w, prefix + "left.", eps, memory.setdefault("left", {}))
    right = hgrn2(h, mixer["right"], w, prefix + "right.", eps, memory.setdefault("right", {}), reads_out)
    return 0.5 * (rms_div(left, eps) * W(w, prefix + "left.out") + rms_div(right, eps) * W(w, prefix + "right.out"))


# ------------------------------------------------------------------------------------------ feed-forward
def gated_ff(h, w, prefix):
    gate = h @ W(w, prefix + "gate").T + W(w, prefix + "gate.b")
    up = h @ W(w, prefix + "up").T + W(w, prefix + "up.b")
    return (gelu_tanh(gate) * up) @ W(w, prefix + "down").T + W(w, prefix + "down.b")


# ------------------------------------------------------------------------------------------ the model
def layer_forward(x, positions, layer, w, p, eps, memory, reads_out=None):
    h = norm_one_plus(x, W(w, p + "norm1"), eps)
    if (p + "canon1") in w:
        h = input_conv(h, W(w, p + "canon1"), memory)
    if layer["type"] == "parallel":
        y = parallel_mixer(h, positions, layer["mixer"], w, p + "mix.", eps, memory, reads_out)
    else:
        y = window_attention(h, positions, layer["mixer"], w, p + "mix.", eps, memory)
    x = x + y
    if layer.get("mlp") is not None:
        x = x + gated_ff(norm_one_plus(x, W(w, p + "norm2"), eps), w, p + "mlp.")
    return x


def forward(config, w, tokens, memory=None, start=0, layers_out=None, reads_out=None):
    """Logits [T, vocab] of `tokens` at positions start, start + 1, ... of one sequence; `memory` (a
    dictionary, empty at the sequence's start) carries the layers' keys, values and states from call to
    call.  layers_out, if a list, receives the residual stream after every run of a layer; reads_out, if a list,
    what hgrn2 reports of every run of a recurrent layer."""
    memory = {} if memory is None else memory
    eps = float(config["norm"]["eps"])
    positions = list(range(start, start + len(tokens)))
    x0 = embed(tokens, w, eps)
    x = x0
    loop = config.get("loop")
    for i, t in run_order(len(config["layers"]), loop):
        if loop and i == int(loop["start"]):
            x = loop_entry(x, x0, w, t)
        x = layer_forward(x, positions, config["layers"][i], w, "l%d." % i, eps, memory.setdefault((i, t), {}), reads_out)
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm_one_plus(x, W(w, "final.norm"), eps) @ W(w, "embed").T
