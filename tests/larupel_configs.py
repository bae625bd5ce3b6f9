"""Tiny Larupel configurations for the tests.  They differ in every size and option: the order of
the three mixers, heads and kv heads (equal, or one kv head for all), key and value sizes (equal
or not, sizes the matrix-core kernels take or odd ones), convolution taps (down to 2), dense,
routed and absent feed-forwards, one expert chosen, several or all, with and without a shared
expert, and which attention layer lends its keys and values to which."""


def attention(heads, kv_heads, dim, vdim, scale, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return "attention", m


def delta(heads, kv_heads, dim, vdim, conv):
    return "delta", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def general_delta(heads, dim):
    return "general_delta", {"heads": heads, "dim": dim}


def layer(mixer, mlp):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def model(vocab, width, eps, layers):
    return {"architecture": "Larupel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


# values longer than keys; the last layer reads the first layer's keys and values
L_A = model(200, 64, 1e-5, [
    layer(attention(4, 2, 16, 24, 0.2), dense(96)),
    layer(general_delta(2, 16), moe(24, 6, 2, shared=40)),
    layer(delta(4, 2, 16, 8, 3), moe(20, 4, 4)),
    layer(attention(4, 2, 16, 24, 0.2, kv_from=0), dense(48)),
])

# nothing divides by four; a layer without a feed-forward; one kv head for three heads; keys longer
# than values; two taps; one expert of five; two lending layers
L_B = model(131, 50, 3e-6, [
    layer(delta(3, 3, 7, 9, 2), None),
    layer(attention(3, 1, 10, 6, 0.31), moe(30, 5, 1, shared=22)),
    layer(general_delta(5, 6), dense(70)),
    layer(attention(2, 2, 12, 12, 0.25), None),
    layer(attention(3, 1, 10, 6, 0.4, kv_from=1), moe(14, 3, 3)),
    layer(general_delta(1, 20), moe(16, 7, 2, shared=9)),
    layer(attention(2, 2, 12, 12, 0.3, kv_from=3), dense(33)),
])

# sizes that the matrix-core kernels take; a recurrent layer first
L_C = model(384, 128, 1e-6, [
    layer(general_delta(2, 64), dense(256)),
    layer(attention(4, 2, 64, 64, 0.125), moe(64, 8, 3, shared=128)),
    layer(delta(4, 2, 32, 64, 4), moe(64, 8, 2, shared=64)),
    layer(attention(4, 2, 64, 64, 0.125, kv_from=1), dense(128)),
    layer(delta(2, 1, 64, 32, 5), dense(128)),
])

STD = 0.08
ALL = {"A": (L_A, 16, 11), "B": (L_B, 4, 12), "C": (L_C, 16, 13)}      # configuration, page size, seed
