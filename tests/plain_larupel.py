"""A plain, slow implementation of the Larupel decoder: whole sequences, no cache, one function
for each mechanism, float64 on the CPU.  It shares no code with the engine under
``lucciola_amd`` and is what the engine is compared with.

Notation: x is the residual stream [T, width]; a linear weight is stored [out, in] and applied
as W x; positions count from 0; a layer's tensors are named ``l<i>.`` + what the functions below
look up.
"""
import math

import torch

F64 = torch.float64


def linear(x, weight):
    """y[t, n] = sum_k x[t, k] W[n, k]"""
    return x.to(F64) @ weight.to(F64).T


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z.to(F64)))


def silu(z):
    return z.to(F64) * sigmoid(z)


def softplus(z):
    z = z.to(F64)
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def gelu_tanh(z):
    z = z.to(F64)
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last dimension (eps inside the root)."""
    x = x.to(F64)
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def unit_length(x, eps=1e-6):
    """x / sqrt(sum(x^2) + eps) over the last dimension."""
    x = x.to(F64)
    return x / torch.sqrt((x * x).sum(dim=-1, keepdim=True) + eps)


def layer_norm(x, weight, bias, eps):
    """(x - mean) / sqrt(mean of squared deviations + eps) * w + b over the last dimension."""
    x = x.to(F64)
    mean = x.mean(dim=-1, keepdim=True)
    dev = x - mean
    var = (dev * dev).mean(dim=-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * weight.to(F64) + bias.to(F64)


def sinusoid(positions, width):
    """[T, width]: entry 2i is sin(p f_i), entry 2i + 1 cos(p f_i), f_i = 10000^(-2i/width)."""
    p = torch.as_tensor(positions, dtype=F64)[:, None]
    out = torch.zeros((p.shape[0], width), dtype=F64)
    i = torch.arange((width + 1) // 2, dtype=F64)
    angle = p * torch.pow(torch.tensor(10000.0, dtype=F64), -2.0 * i / width)[None, :]
    out[:, 0::2] = torch.sin(angle)
    out[:, 1::2] = torch.cos(angle)[:, :width // 2]
    return out


def embed(weights, ids, first_position=0):
    table = weights["embed"].to(F64)
    x = table[torch.as_tensor(ids, dtype=torch.long)]
    return x + sinusoid(range(first_position, first_position + len(ids)), table.shape[1])


# ------------------------------------------------------------------------------ mixers
def softmax_attention(q, k, v, scale, temp):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; head h reads key/value head h // (H / G); row i sees
    columns j <= i; score (q . k) scale temp[h]."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros((T, H, v.shape[2]), dtype=F64)
    seen = torch.tril(torch.ones((T, T), dtype=torch.bool))
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale * float(temp[h])
        s = s.masked_fill(~seen, -math.inf)
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def attention_keys_values(h, weights, p, m, eps):
    """What an attention layer caches: its normed keys [T, G, d] and its values [T, G, dv]."""
    T = h.shape[0]
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = linear(h, weights[p + "k"]).view(T, G, d)
    k = unit_rms(k, eps) * weights[p + "k.norm"].to(F64)
    v = linear(h, weights[p + "v"]).view(T, G, dv)
    return k, v


def attention_mixer(h, weights, p, m, eps, kv):
    """``kv``: the keys and values this layer reads (its own or another layer's)."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    q = linear(h, weights[p + "q"]).view(T, H, d)
    q = unit_rms(q, eps) * weights[p + "q.norm"].to(F64)
    k, v = kv
    o = softmax_attention(q, k, v, float(m["scale"]), weights[p + "temp"].to(F64))
    return linear(o.reshape(T, -1), weights[p + "o"])


def causal_conv(x, taps):
    """x [T, C], taps [C, K]: y[t, c] = sum_j taps[c, K - 1 - j] x[t - j, c], zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    x, taps = x.to(F64), taps.to(F64)
    padded = torch.cat([torch.zeros((K - 1, C), dtype=F64), x], dim=0)
    y = torch.zeros((T, C), dtype=F64)
    for j in range(K):
        y += padded[K - 1 - j:K - 1 - j + T] * taps[:, K - 1 - j][None, :]
    return y


def gated_delta_mixer(h, weights, p, m, eps):
    """Per head, token by token: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(linear(h, weights[p + "q"]), weights[p + "q.conv"])).view(T, G, d)
    k = silu(causal_conv(linear(h, weights[p + "k"]), weights[p + "k.conv"])).view(T, G, d)
    v = silu(causal_conv(linear(h, weights[p + "v"]), weights[p + "v.conv"])).view(T, H, dv)
    q = unit_length(q) * d ** -0.5
    k = unit_length(k)
    beta = sigmoid(linear(h, weights[p + "b"]))                                   # [T, H]
    rate = torch.exp(weights[p + "A_log"].to(F64))[None, :] * softplus(linear(h, weights[p + "a"])
                                                                      + weights[p + "dt_bias"].to(F64))
    g = torch.exp(-rate)                                                          # [T, H]
    out = torch.zeros((T, H, dv), dtype=F64)
    for head in range(H):
        kv = head // (H // G)
        S = torch.zeros((d, dv), dtype=F64)
        for t in range(T):
            S = g[t, head] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            out[t, head] = S.T @ q[t, kv]
    out = unit_rms(out, eps) * weights[p + "norm"].to(F64)                        # weight [dv], shared by heads
    gate = silu(linear(h, weights[p + "g"])).view(T, H, dv)
    return linear((out * gate).reshape(T, -1), weights[p + "o"])


def general_delta_mixer(h, weights, p, m, eps):
    """Per head, token by token, with the unit key u = k / sqrt(sum k^2 + 1e-6):
    S <- diag(w) S - (a u)(u^T S) + k v^T (u^T S is taken of S before its decay); o = S^T r."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    r = linear(h, weights[p + "r"]).view(T, H, d)
    k = linear(h, weights[p + "k"]).view(T, H, d)
    v = linear(h, weights[p + "v"]).view(T, H, d)
    inner = torch.tanh(linear(h, weights[p + "w1"]))
    w = torch.exp(-math.exp(-0.5) * sigmoid(linear(inner, weights[p + "w2"]) + weights[p + "w0"].to(F64)))
    w = w.view(T, H, d)
    a = sigmoid(linear(h, weights[p + "a"]) + weights[p + "a.b"].to(F64)).view(T, H, d)
    u = unit_length(k)
    out = torch.zeros((T, H, d), dtype=F64)
    for head in range(H):
        S = torch.zeros((d, d), dtype=F64)
        for t in range(T):
            uS = u[t, head] @ S                                                   # [dv]
            S = w[t, head][:, None] * S - torch.outer(a[t, head] * u[t, head], uS) \
                + torch.outer(k[t, head], v[t, head])
            out[t, head] = S.T @ r[t, head]
    out = unit_rms(out, eps).reshape(T, -1) * weights[p + "norm"].to(F64)        # weight [H d]
    return linear(out * sigmoid(linear(h, weights[p + "g"])), weights[p + "o"])


# ------------------------------------------------------------------------------ feed-forwards
def gated_ff(h, weights, p, act):
    return linear(act(linear(h, weights[p + "gate"])) * linear(h, weights[p + "up"]), weights[p + "down"])


def routed_ff(h, weights, p, mlp):
    """Router logits z = W h + b; the ``top`` largest are chosen, their weights are the softmax over
    the chosen logits alone; a shared expert, where there is one, runs for every token and is
    added times sigmoid(w_sg . h)."""
    T = h.shape[0]
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    z = linear(h, weights[p + "router"]) + weights[p + "router.b"].to(F64)
    out = torch.zeros((T, h.shape[1]), dtype=F64)
    outputs = [gated_ff(h, weights, p + f"e{e}.", silu) for e in range(E)]
    for t in range(T):
        order = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        share = torch.softmax(z[t, order], dim=0)
        for n, e in enumerate(order):
            out[t] += share[n] * outputs[e][t]
    if mlp.get("shared"):
        gate = sigmoid(linear(h, weights[p + "shared.sg"]))                        # [T, 1]
        out = out + gate * gated_ff(h, weights, p + "shared.", silu)
    return out


def feed_forward(h, weights, p, mlp):
    if mlp["kind"] == "dense":
        return gated_ff(h, weights, p, gelu_tanh)
    return routed_ff(h, weights, p, mlp)


# ------------------------------------------------------------------------------ the model
def norm_of(weights, name, x, eps):
    return layer_norm(x, weights[name], weights[name + ".b"], eps)


def forward(cfg, weights, ids, streams=None):
    """Logits [T, vocab] of a whole sequence.  ``streams``: a list that receives the residual
    stream after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = embed(weights, ids)
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = norm_of(weights, p + "norm1", x, eps)
        if layer["type"] == "attention":
            if m.get("kv_from") is None:
                kept[i] = attention_keys_values(h, weights, p + "mix.", m, eps)
                kv = kept[i]
            else:
                kv = kept[int(m["kv_from"])]
            y = attention_mixer(h, weights, p + "mix.", m, eps, kv)
        elif layer["type"] == "delta":
            y = gated_delta_mixer(h, weights, p + "mix.", m, eps)
        elif layer["type"] == "general_delta":
            y = general_delta_mixer(h, weights, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + norm_of(weights, p + "norm1b", y, eps)
        if layer.get("mlp"):
            h = norm_of(weights, p + "norm2", x, eps)
            x = x + norm_of(weights, p + "norm2b", feed_forward(h, weights, p + "mlp.", layer["mlp"]), eps)
        if streams is not None:
            streams.append(x.clone())
    return linear(norm_of(weights, "final.norm", x, eps), weights["head"])


def greedy(cfg, weights, prompt, new_tokens):
    """Greedy generation by running the whole sequence again for every token; ties go to the
    lowest index."""
    ids, out = list(prompt), []
    for _ in range(new_tokens):
        tok = int(torch.argmax(forward(cfg, weights, ids)[-1]))
        out.append(tok)
        ids.append(tok)
    return out
