"""A plain, slow implementation of the Pubodra decoder: whole sequences, no cache, one function
for each mechanism, float64 on the CPU.  It shares no code with the engine under
``lucciola_amd`` and is what the engine is compared with.

Notation: x is the residual stream [T, width]; a linear weight is stored [out, in] and applied
as W x; positions count from 0.
"""
import math

import torch

F64 = torch.float64


def linear(x, weight):
    """y[t, n] = sum_k x[t, k] W[n, k]"""
    return x.to(F64) @ weight.to(F64).T


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last dimension (eps inside the root)."""
    x = x.to(F64)
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def dynamic_tanh(x, weight, bias, alpha):
    """tanh(alpha x) w + b: a norm that takes no mean and no variance."""
    return torch.tanh(float(alpha) * x.to(F64)) * weight.to(F64) + bias.to(F64)


def gelu_tanh(z):
    z = z.to(F64)
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def relu_squared(z):
    return torch.clamp(z.to(F64), min=0.0) ** 2


def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims), i < dims/2, and the factor on cosines and sines.  With YaRN
    scaling (factor, original, fast, slow): a frequency is divided by ``factor`` to the degree
    ramp_i that its wavelength is long against the original context."""
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    f = torch.pow(torch.tensor(float(base), dtype=F64), -2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    f = f / factor * ramp + f * (1.0 - ramp)
    return f, 0.1 * math.log(factor) + 1.0


def rotate_interleaved(x, positions, dims, base, scaling=None):
    """x: [T, ..., n].  Of the last dimension's first ``dims`` entries, entry 2i pairs with
    entry 2i + 1: (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = position * f_i; the rest
    pass unchanged."""
    x = x.to(F64).clone()
    f, mag = rotary_frequencies(dims, base, scaling)
    angle = torch.as_tensor(positions, dtype=F64)[:, None] * f[None, :]     # [T, dims/2]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    cos, sin = (torch.cos(angle) * mag).view(shape), (torch.sin(angle) * mag).view(shape)
    u, v = x[..., 0:dims:2].clone(), x[..., 1:dims:2].clone()
    x[..., 0:dims:2] = u * cos - v * sin
    x[..., 1:dims:2] = v * cos + u * sin
    return x


def windowed_softmax(scores, positions, window):
    """scores [T, T] of one head; row i sees column j where 0 <= p_i - p_j (< window)."""
    pos = torch.as_tensor(positions, dtype=torch.long)
    diff = pos[:, None] - pos[None, :]
    seen = diff >= 0
    if window:
        seen &= diff < window
    s = scores.masked_fill(~seen, float("-inf"))
    s = s - s.max(dim=-1, keepdim=True).values
    p = torch.exp(s)
    return p / p.sum(dim=-1, keepdim=True)


def latent_attention(h, w, m, positions, eps):
    """The mixer.  ``w``: its tensors by short name (q, dkv, dkv.norm, uk, uv, g, o); ``m``:
    its sizes and constants (heads, dim, rot_dim, vdim, kv_rank, scale, rot, mask)."""
    H, dim, rot_dim, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    rot = m.get("rot") or {}
    q = linear(h, w["q"]).view(T, H, dim + rot_dim)
    q_plain, q_turn = q[..., :dim], q[..., dim:]
    down = linear(h, w["dkv"])
    latent = unit_rms(down[:, :rank], eps) * w["dkv.norm"].to(F64)
    k_turn = down[:, rank:].view(T, 1, rot_dim)
    if rot:
        q_turn = rotate_interleaved(q_turn, positions, rot["dims"], rot["base"], rot.get("scaling"))
        k_turn = rotate_interleaved(k_turn, positions, rot["dims"], rot["base"], rot.get("scaling"))
    k_plain = linear(latent, w["uk"]).view(T, H, dim)
    value = linear(latent, w["uv"]).view(T, H, vdim)
    window = (m.get("mask") or {}).get("size")
    out = torch.zeros(T, H, vdim, dtype=F64)
    for head in range(H):
        s = (q_plain[:, head] @ k_plain[:, head].T + q_turn[:, head] @ k_turn[:, 0].T) * float(m["scale"])
        out[:, head] = windowed_softmax(s, positions, window) @ value[:, head]
    gate = torch.sigmoid(linear(h, w["g"]))
    return linear(out.reshape(T, H * vdim) * gate, w["o"])


def dense_feed_forward(h, w):
    return linear(gelu_tanh(linear(h, w["up"])), w["down"])


def routed_feed_forward(h, w, experts, top):
    """Scores are a softmax over all experts; the ``top`` largest are kept and their scores
    divided by their sum (+ 1e-20); the experts' outputs are added with those weights."""
    T = h.shape[0]
    scores = torch.softmax(linear(h, w["router"]), dim=-1)
    picked, chosen = torch.topk(scores, top, dim=-1)
    weights = picked / (picked.sum(dim=-1, keepdim=True) + 1e-20)
    out = torch.zeros(T, h.shape[1], dtype=F64)
    for t in range(T):
        for k in range(top):
            e = int(chosen[t, k])
            y = linear(relu_squared(linear(h[t:t + 1], w[f"e{e}.up"])), w[f"e{e}.down"])
            out[t] += weights[t, k] * y[0]
    return out


def _sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def _norm(x, weights, name):
    return dynamic_tanh(x, weights[name], weights[name + ".b"], float(weights[name + ".alpha"]))


def layer(x, cfg, weights, index, positions):
    entry = cfg["layers"][index]
    eps = cfg["norm"]["eps"]
    p = f"l{index}."
    if entry["type"] != "latent_attention":
        raise ValueError(entry["type"])
    x = x + latent_attention(_norm(x, weights, p + "norm1"), _sub(weights, p + "mix."), entry["mixer"],
                             positions, eps)
    mlp = entry.get("mlp")
    if mlp:
        h = _norm(x, weights, p + "norm2")
        if mlp["kind"] == "dense":
            x = x + dense_feed_forward(h, _sub(weights, p + "mlp."))
        else:
            x = x + routed_feed_forward(h, _sub(weights, p + "mlp."), mlp["router"]["experts"],
                                        mlp["router"]["top"])
    return x


def run_order(cfg):
    """(layer, pass number or None) in the order they run: the layers of the loop ``times``
    times in a row, the others once."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    order = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        order += [(i, t) for i in range(loop["start"], loop["stop"])]
    return order + [(i, None) for i in range(loop["stop"], n)]


def forward(cfg, weights, ids, positions=None, trace=None):
    """Logits [T, vocab] of one sequence.  ``trace``: a list that receives the stream after every
    layer run."""
    T = len(ids)
    positions = list(range(T)) if positions is None else positions
    x = weights["embed"][torch.as_tensor(ids, dtype=torch.long)].to(F64)
    loop = cfg.get("loop")
    for index, turn in run_order(cfg):
        if turn is not None and index == loop["start"]:
            x = x + weights["loop.step"][turn].to(F64)
        x = layer(x, cfg, weights, index, positions)
        if trace is not None:
            trace.append(x.clone())
    return linear(_norm(x, weights, "final.norm"), weights["embed"])


def greedy(cfg, weights, prompt, new_tokens):
    """Greedy generation by running the whole sequence again for every token; ties go to the
    lowest index."""
    ids, out = list(prompt), []
    for _ in range(new_tokens):
        tok = int(torch.argmax(forward(cfg, weights, ids)[-1]))
        out.append(tok)
        ids.append(tok)
    return out
