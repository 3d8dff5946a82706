"""Small Bovozen configurations (config.json dictionaries) for the tests.  They differ from each other in every
size: head counts and groups of the attention and of the delta rule, key and value sizes that differ inside a layer
(either may be the larger), scales that are not 1/sqrt of anything, blocks of 1, 5, 7, 20, 64, 65 and 70 positions
and none, convolutions of 1 to 5 taps, low-rank sizes of 1 to 40, layers with and without blending and feed-forward,
delta layers first, last and alone, experts with top = 1 and top = all, with and without a shared expert, sizes that
are multiples of nothing."""


def attn(heads, kv_heads, dim, vdim, scale, block=None, v_mix=False):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if block:
        m["mask"] = {"size": block}
    if v_mix:
        m["v_mix"] = True
    return {"type": "attention", "mixer": m}


def delta(heads, kv_heads, dim, vdim, conv, decay_rank=4, gate_rank=6):
    return {"type": "channel_delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                                               "decay_rank": decay_rank, "gate_rank": gate_rank}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def model(vocab, width, eps, max_positions, layers):
    return {"architecture": "Bovozen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "max_positions": max_positions,
            "layers": layers}


MIXED = model(173, 72, 1e-6, 700, [
    layer(delta(4, 2, 8, 12, 4), dense(88)),
    layer(attn(6, 2, 8, 20, 0.3, block=20, v_mix=True), moe(5, 2, 24, shared=40)),
    layer(attn(2, 2, 24, 8, 0.2), None),
    layer(attn(4, 2, 12, 20, 0.25, block=70, v_mix=True), moe(3, 3, 16)),
    layer(delta(1, 1, 20, 7, 2, decay_rank=1, gate_rank=3), moe(4, 1, 40, shared=8)),
    layer(attn(3, 1, 16, 16, 0.15, block=5), dense(40)),
    layer(attn(2, 2, 4, 20, 0.5, block=33, v_mix=True), dense(24)),
])

BLOCKS = model(97, 48, 1e-5, 600, [
    layer(attn(2, 1, 8, 8, 0.3, block=1, v_mix=True), dense(40)),
    layer(attn(2, 2, 8, 12, 0.2, block=64), dense(56)),
    layer(delta(2, 2, 12, 8, 3), None),
    layer(attn(3, 1, 4, 8, 0.25, block=65, v_mix=True), moe(5, 2, 16, shared=24)),
    layer(attn(1, 1, 16, 16, 0.5, block=7), dense(24)),
])

# sizes that are multiples of nothing; a group of more than 16 query heads; heads wider than the matrix-core kernels
# take; a convolution of one tap (which keeps nothing) and one of five; low-rank sizes above the padding's step
ODD = model(131, 50, 1e-5, 300, [
    layer(attn(3, 3, 5, 9, 0.37, block=9), moe(1, 1, 14, shared=5)),
    layer(delta(6, 2, 3, 5, 1, decay_rank=33, gate_rank=40), dense(13)),
    layer(attn(17, 1, 6, 4, 0.21), moe(7, 3, 10)),
    layer(attn(1, 1, 144, 24, 0.05, block=40), None),
    layer(delta(1, 1, 64, 200, 5, decay_rank=2, gate_rank=1), None),
])

# one mechanism at a time
ONLY_DELTA = model(64, 32, 1e-5, 400, [layer(delta(2, 1, 8, 6, 3), None)])
ONLY_ATTN = model(64, 32, 1e-5, 400, [layer(attn(2, 1, 8, 6, 0.3, block=7), None)])
ONLY_FULL = model(64, 32, 1e-5, 400, [layer(attn(4, 2, 8, 8, 0.3), None)])
ONLY_BLEND = model(64, 32, 1e-5, 400, [layer(attn(2, 1, 8, 8, 0.3, v_mix=True), None),
                                       layer(attn(2, 1, 8, 8, 0.3, block=11, v_mix=True), None)])
ONLY_WIDE = model(64, 32, 1e-5, 600, [layer(attn(2, 1, 8, 8, 0.3, block=150), None)])
ONLY_MOE = model(64, 32, 1e-5, 400, [layer(delta(1, 1, 4, 4, 2), moe(6, 2, 16, shared=12))])

ALL = {"mixed": MIXED, "blocks": BLOCKS, "odd": ODD, "only_delta": ONLY_DELTA, "only_attn": ONLY_ATTN,
       "only_full": ONLY_FULL, "only_blend": ONLY_BLEND, "only_wide": ONLY_WIDE, "only_moe": ONLY_MOE}
