"""Small Rekirax configurations (config.json dictionaries) for the tests.  They differ from each other in every size:
head counts and groups, key and value sizes that differ inside a layer, rotations of all, some and none of a head's
elements, scales that are not 1/sqrt of anything, windows and chunks of 1 to 150 positions and none, caps and none,
convolutions of 1 to 5 taps and none, loops over the first, the middle, the last and all layers, walked once to three
times, and none, layers without feed-forward, sizes that are multiples of nothing."""


def win(heads, kv_heads, dim, scale, window=None, softcap=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if softcap:
        m["softcap"] = softcap
    return {"type": "attention", "mixer": m}


def par(heads, kv_heads, dim, vdim, scale, chunk=None, rot=None, base=10000.0, right=(2, 8, 12)):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if chunk:
        left["mask"] = {"size": chunk}
    if rot:
        left["rot"] = {"dims": rot, "base": base}
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": right[0], "dim": right[1], "vdim": right[2]}}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def model(vocab, width, eps, layers, taps=None, loop=None):
    d = {"architecture": "Rekirax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if taps:
        d["canon"] = {"taps": taps}
    if loop:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return d


MIXED = model(173, 72, 1e-6, [
    layer(par(6, 2, 8, 12, 0.3, chunk=20, rot=4, right=(3, 8, 20)), dense(88)),
    layer(win(4, 2, 24, 0.2, window=33, softcap=5.0), None),
    layer(par(2, 2, 16, 8, 0.25, chunk=70, rot=16, base=500.0, right=(1, 20, 7)), dense(40)),
    layer(win(3, 1, 16, 0.15, window=9, softcap=12.0), dense(24)),
    layer(par(4, 1, 12, 20, 0.35, chunk=5, right=(2, 4, 36)), dense(56)),
], taps=3, loop=(1, 4, 3))

WINDOWS = model(97, 48, 1e-5, [
    layer(win(2, 1, 8, 0.3, window=1), dense(40)),
    layer(win(2, 2, 16, 0.2, window=64, softcap=3.0), dense(56)),
    layer(win(3, 1, 4, 0.25, window=65), None),
    layer(win(1, 1, 16, 0.5, window=7, softcap=30.0), dense(24)),
    layer(win(4, 2, 12, 0.4), dense(16)),
    layer(win(2, 1, 32, 0.1, window=70, softcap=8.0), dense(24)),
], taps=2)

CHUNKS = model(131, 64, 1e-5, [
    layer(par(2, 1, 8, 8, 0.3, chunk=1, rot=8, right=(2, 8, 8)), dense(40)),
    layer(par(4, 2, 16, 12, 0.2, chunk=64, rot=2, base=77.0, right=(1, 32, 64)), None),
    layer(par(3, 3, 4, 8, 0.25, chunk=65, right=(4, 4, 4)), dense(30)),
    layer(par(2, 1, 32, 16, 0.15, chunk=7, rot=32, base=1e6, right=(2, 16, 20)), dense(24)),
    layer(par(1, 1, 16, 16, 0.5, right=(1, 64, 40)), dense(16)),
], taps=4, loop=(0, 5, 1))

ODD = model(61, 50, 3e-6, [
    layer(par(3, 1, 10, 6, 0.21, chunk=9, rot=6, right=(3, 5, 9)), dense(37)),
    layer(win(5, 5, 6, 0.33, window=11, softcap=2.5), dense(29)),
    layer(par(2, 2, 18, 22, 0.11, chunk=33, rot=10, base=3000.0, right=(1, 7, 33)), dense(13)),
], taps=5, loop=(2, 3, 2))

PLAIN = model(80, 32, 1e-5, [                     # no convolution, no loop
    layer(win(2, 1, 16, 0.25, window=20, softcap=10.0), dense(48)),
    layer(par(2, 2, 16, 16, 0.25, chunk=16, rot=8, right=(2, 8, 16)), dense(48)),
])

# heads of the sizes the matrix-core attention and the wave-a-token packing kernel are built for, a chunk and a window that
# cross pages, recurrent heads of 32 channels
MEDIUM = model(500, 256, 1e-5, [
    layer(par(4, 2, 64, 64, 0.11, chunk=100, rot=32, base=250000.0, right=(4, 32, 48)), dense(512)),
    layer(win(4, 1, 128, 0.09, window=200, softcap=20.0), dense(384)),
    layer(par(8, 8, 32, 32, 0.18, chunk=64, rot=32, right=(2, 64, 32)), dense(512)),
    layer(par(4, 2, 64, 64, 0.14, chunk=130, rot=24, right=(3, 32, 80)), None),
], taps=4, loop=(1, 3, 2))

# one mechanism at a time
ONLY_WINDOW = model(90, 40, 1e-5, [layer(win(2, 1, 16, 0.4, window=7, softcap=20.0), dense(32))], taps=1)
ONLY_WIDE_WINDOW = model(90, 40, 1e-5, [layer(win(2, 2, 32, 0.3, window=150, softcap=20.0), None)], taps=1)
ONLY_CHUNK = model(90, 40, 1e-5, [layer(par(2, 1, 16, 16, 0.4, chunk=7, rot=4, right=(1, 4, 4)), dense(32))], taps=1)
ONLY_WIDE_CHUNK = model(90, 40, 1e-5, [layer(par(2, 2, 32, 32, 0.3, chunk=150, rot=32, right=(1, 4, 4)), None)], taps=1)
# the attention of this one sees the token itself only: earlier tokens reach a position through the recurrence alone
ONLY_STATE = model(90, 40, 1e-5, [layer(par(2, 1, 8, 8, 0.4, chunk=1, right=(2, 16, 24)), dense(32))], taps=1)
# and here through the convolution alone
ONLY_CONV = model(90, 40, 1e-5, [layer(win(2, 1, 8, 0.4, window=1), dense(32))], taps=4)
ONLY_FULL = model(90, 48, 1e-5, [layer(win(2, 1, 64, 0.2, softcap=40.0), dense(32))], taps=2)
LOOPED = model(90, 40, 1e-5, [layer(par(2, 1, 8, 8, 0.4, chunk=12, rot=8, right=(2, 8, 8)), dense(32))], taps=2, loop=(0, 1, 3))

ALL = {"mixed": MIXED, "medium": MEDIUM, "windows": WINDOWS, "chunks": CHUNKS, "odd": ODD, "plain": PLAIN, "only_window": ONLY_WINDOW,
       "only_wide_window": ONLY_WIDE_WINDOW, "only_chunk": ONLY_CHUNK, "only_wide_chunk": ONLY_WIDE_CHUNK,
       "only_state": ONLY_STATE, "only_conv": ONLY_CONV, "only_full": ONLY_FULL, "looped": LOOPED}
