"""A plain, slow implementation of the Bovozen design in float64 torch on the CPU: one function per
mechanism, written from the design's equations and sharing nothing with yalm_amd.  The tests hold the
library against it.

The design: a decoder whose token embedding gets a learned position vector, whose layers are pre-norm
(x <- x + mixer(n1(x)); x <- x + ff(n2(x)), the norms' weights stored as their distance from one), whose
mixers are a grouped-query attention without rotation (norms over the whole query and key projections, a
slope per head times the distance, keys visible inside the query's own block of positions only, values
blended with those of the first such layer) or a gated delta rule with a decay for every key channel
(short convolutions in front, unit queries and keys, a low-rank decay and a low-rank output gate), and
whose feed-forwards are a two-matrix layer with the erf gelu or a mixture of gated experts beside a
shared expert with a gate of its own.  The head is the embedding table.

`weights` is a dictionary name -> tensor with the names of a model folder ('l3.mix.q', ...).  `memory`,
where a function takes one, is what the layers keep of earlier tokens of ONE sequence: a dictionary the
functions fill and read, so that a text can be fed in pieces."""
import math

import torch

F64 = torch.float64
UNIT_FLOOR = 1e-6                # under the root of a unit vector's sum of squares
SLOPE_EXPONENT = 8.0


def W(w, name):
    return w[name].to(F64)


def rms_div(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def norm_one_plus(x, w_around_zero, eps):
    """The layers' norm: the stored weight is the distance from one."""
    return rms_div(x, eps) * (1.0 + w_around_zero)


def silu(z):
    return z * torch.sigmoid(z)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


# ------------------------------------------------------------------------------------------ embedding
def embed(tokens, positions, w):
    return W(w, "embed")[torch.tensor(tokens, dtype=torch.long)] + W(w, "pos")[torch.tensor(positions, dtype=torch.long)]


# ------------------------------------------------------------------------------------------ attention
def head_slopes(H):
    return [2.0 ** (-SLOPE_EXPONENT * (i + 1) / H) for i in range(H)]


def visible(i, j, block):
    """Whether the query at position i sees the key at position j (block 0: every earlier key)."""
    return j <= i and (not block or i // block == j // block)


def attention(h, positions, mixer, w, prefix, eps, memory, v_first=None):
    """One attention mixer over the rows of h at `positions` (consecutive), with what `memory` holds of the
    sequence's earlier keys and values ({'k': [S, G, d], 'v': [S, G, dv]}, from position 0 on).  v_first
    [T, G, dv]: the values of the first blending layer for the same tokens (None for that layer itself, or
    without blending).  Returns ([T, width], the values as this layer remembers them [T, G, dv])."""
    H, G, d, dv = int(mixer["heads"]), int(mixer["kv_heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q = rms_div(h @ W(w, prefix + "q").T, eps) * W(w, prefix + "q.norm")
    k = rms_div(h @ W(w, prefix + "k").T, eps) * W(w, prefix + "k.norm")
    v = (h @ W(w, prefix + "v").T).reshape(T, G, dv)
    q, k = q.reshape(T, H, d), k.reshape(T, G, d)
    if v_first is not None:
        lam = float(W(w, prefix + "vmix"))
        v = (1.0 - lam) * v + lam * v_first
    keys = torch.cat([memory["k"], k]) if "k" in memory else k
    values = torch.cat([memory["v"], v]) if "v" in memory else v
    memory["k"], memory["v"] = keys, values
    assert keys.shape[0] == positions[-1] + 1
    scale = float(mixer["scale"])
    block = int(mixer["mask"]["size"]) if mixer.get("mask") else 0
    slopes = head_slopes(H)
    out = torch.zeros((T, H, dv), dtype=F64)
    for t, p in enumerate(positions):
        js = [j for j in range(p + 1) if visible(p, j, block)]
        idx = torch.tensor(js, dtype=torch.long)
        dist = p - idx.to(F64)
        for hd in range(H):
            g = hd // (H // G)
            s = (keys[idx, g] @ q[t, hd]) * scale - slopes[hd] * dist
            out[t, hd] = torch.softmax(s, dim=0) @ values[idx, g]
    return out.reshape(T, H * dv) @ W(w, prefix + "o").T, v


# ------------------------------------------------------------------------------------------ delta rule
def short_conv(x, taps_w, before):
    """y[t, c] = sum_j taps_w[c, j] x[t - (n - 1) + j, c] with n taps, the last tap on the token itself; `before`
    [n - 1, C] are the inputs in front of x (zeros at a sequence's start).  Returns (y, the last n - 1 inputs)."""
    n = taps_w.shape[1]
    full = torch.cat([before, x])
    y = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for j in range(n):
            y[t] += taps_w[:, j] * full[t + j]
    return y, full[full.shape[0] - (n - 1):]


def unit(x):
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + UNIT_FLOOR)


def delta_inputs(h, mixer, w, prefix, memory):
    """What the recurrence takes in for the rows of h: q [T, Gq, d] (unit, times d^-1/2), k [T, Gq, d] (unit),
    v [T, H, dv], beta [T, H], decay [T, H, d]."""
    H, G, d, dv = int(mixer["heads"]), int(mixer["kv_heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    outs = {}
    for name, C in (("q", G * d), ("k", G * d), ("v", H * dv)):
        taps_w = W(w, prefix + name + ".conv")
        before = memory.get("conv." + name)
        if before is None:
            before = torch.zeros((taps_w.shape[1] - 1, C), dtype=F64)
        y, memory["conv." + name] = short_conv(h @ W(w, prefix + name).T, taps_w, before)
        outs[name] = silu(y)
    q = unit(outs["q"].reshape(T, G, d)) * d ** -0.5
    k = unit(outs["k"].reshape(T, G, d))
    v = outs["v"].reshape(T, H, dv)
    beta = torch.sigmoid(h @ W(w, prefix + "b").T)
    step = torch.nn.functional.softplus((h @ W(w, prefix + "a1").T) @ W(w, prefix + "a2").T + W(w, prefix + "dt_bias"))
    decay = torch.exp(-torch.exp(W(w, prefix + "A_log"))[None, :, None] * step.reshape(T, H, d))
    return q, k, v, beta, decay


def delta_recurrence(q, k, v, beta, decay, S):
    """S [H, d, dv] -> (o [T, H, dv], S): per head S <- decay * S (row by row); u = beta (v - S^T k); S <- S + k u^T;
    o = S^T q.  Head h reads the query/key head h // (H / Gq)."""
    T, H, dv = v.shape
    rep = H // q.shape[1]
    o = torch.zeros((T, H, dv), dtype=F64)
    for t in range(T):
        for hd in range(H):
            kk, qq = k[t, hd // rep], q[t, hd // rep]
            S[hd] = decay[t, hd][:, None] * S[hd]
            u = beta[t, hd] * (v[t, hd] - S[hd].T @ kk)
            S[hd] = S[hd] + kk[:, None] * u[None, :]
            o[t, hd] = S[hd].T @ qq
    return o, S


def channel_delta(h, mixer, w, prefix, eps, memory):
    """The gated delta rule over the rows of h [T, width], from the state in `memory` (made at zero if absent), which
    it leaves advanced.  Returns [T, width]."""
    H, d, dv = int(mixer["heads"]), int(mixer["dim"]), int(mixer["vdim"])
    T = h.shape[0]
    q, k, v, beta, decay = delta_inputs(h, mixer, w, prefix, memory)
    S = memory.get("S")
    if S is None:
        S = torch.zeros((H, d, dv), dtype=F64)
    o, memory["S"] = delta_recurrence(q, k, v, beta, decay, S)
    o = rms_div(o, eps) * W(w, prefix + "norm")
    gate = torch.sigmoid((h @ W(w, prefix + "g1").T) @ W(w, prefix + "g2").T)
    return (o.reshape(T, H * dv) * gate) @ W(w, prefix + "o").T


# ------------------------------------------------------------------------------------------ feed-forwards
def dense_ff(h, w, prefix):
    return gelu_erf(h @ W(w, prefix + "up").T) @ W(w, prefix + "down").T


def gated_ff(h, w, prefix):
    return (silu(h @ W(w, prefix + "gate").T) * (h @ W(w, prefix + "up").T)) @ W(w, prefix + "down").T


def router_logits(h, w, prefix):
    return h @ W(w, prefix + "router").T + W(w, prefix + "router.b")


def route(h, w, prefix, top):
    """(ids [T, top], weights [T, top]): the experts with the largest logits and the softmax over those."""
    vals, ids = torch.topk(router_logits(h, w, prefix), top, dim=-1)
    return ids, torch.softmax(vals, dim=-1)


def route_margin(h, w, prefix, top):
    """Per row, by how much the last chosen logit exceeds the first one left out (inf if all are chosen)."""
    z = router_logits(h, w, prefix)
    if top >= z.shape[-1]:
        return torch.full((z.shape[0],), math.inf, dtype=F64)
    vals, _ = torch.topk(z, top + 1, dim=-1)
    return vals[:, top - 1] - vals[:, top]


def moe_ff(h, mlp, w, prefix):
    top = int(mlp["router"]["top"])
    ids, wts = route(h, w, prefix, top)
    out = torch.zeros((h.shape[0], W(w, prefix + "e0.down").shape[0]), dtype=F64)
    for t in range(h.shape[0]):
        for c in range(top):
            out[t] += wts[t, c] * gated_ff(h[t:t + 1], w, prefix + "e%d." % int(ids[t, c]))[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ W(w, prefix + "shared.sg").T) * gated_ff(h, w, prefix + "shared.")
    return out


def feed_forward(h, mlp, w, prefix):
    if mlp["kind"] == "dense":
        return dense_ff(h, w, prefix)
    return moe_ff(h, mlp, w, prefix)


# ------------------------------------------------------------------------------------------ the model
def forward(config, w, tokens, memory=None, start=0, layers_out=None, margins_out=None):
    """Logits [T, vocab] of `tokens` at positions start, start + 1, ... of one sequence; `memory` (a
    dictionary, empty at the sequence's start) carries the layers' keys, values and states from call to
    call.  layers_out, if a list, receives the residual stream after every layer; margins_out the
    router margins [T] of every mixture layer."""
    memory = {} if memory is None else memory
    eps = float(config["norm"]["eps"])
    positions = list(range(start, start + len(tokens)))
    x = embed(tokens, positions, w)
    v_first = None
    for i, layer in enumerate(config["layers"]):
        p = "l%d." % i
        mem = memory.setdefault(i, {})
        h = norm_one_plus(x, W(w, p + "norm1"), eps)
        mixer = layer["mixer"]
        if layer["type"] == "channel_delta":
            y = channel_delta(h, mixer, w, p + "mix.", eps, mem)
        else:
            blend = bool(mixer.get("v_mix"))
            y, v = attention(h, positions, mixer, w, p + "mix.", eps, mem, v_first if blend else None)
            if blend and v_first is None:
                v_first = v
        x = x + y
        mlp = layer.get("mlp")
        if mlp is not None:
            h = norm_one_plus(x, W(w, p + "norm2"), eps)
            if margins_out is not None and mlp["kind"] == "moe":
                margins_out.append(route_margin(h, w, p + "mlp.", int(mlp["router"]["top"])))
            x = x + feed_forward(h, mlp, w, p + "mlp.")
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm_one_plus(x, W(w, "final.norm"), eps) @ W(w, "embed").T
