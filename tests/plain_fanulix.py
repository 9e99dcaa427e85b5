"""A plain, slow Fanulix in float64 on the CPU: one function per mechanism, whole sequences at once, no cache.
It shares nothing with the engine; the tests compare the engine with it.

cfg is the parsed config.json (a dict), w a dict name -> float64 tensor.
"""
import math

import torch

F = torch.float64


# ---- small functions ---------------------------------------------------------------------------------------------
def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, weight, bias, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * weight + bias


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


# ---- softmax attention with a sink of score zero ------------------------------------------------------------------
def query_temperature(positions, coef, every):
    """1 + coef ln(floor((p + 1) / every) + 1) per position."""
    steps = torch.div(positions + 1, every, rounding_mode="floor")
    return 1.0 + coef * torch.log(steps.to(F) + 1.0)


def softmax_plus_one(scores, mask):
    """exp(s_j) / (1 + sum over the visible exp(s_j)): a sink of score 0 that has no value."""
    s = scores.masked_fill(~mask, float("-inf"))
    m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(-1, keepdim=True))


def sink_attention(h, w, p, m, eps, positions):
    """h [T, width]; tensors p + 'q', 'k', 'v' (with '.b'), 'g', 'o'; m the sizes and constants of the mixer's side."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(T, H, D)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(T, G, D)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(T, G, V)
    q, k = rms_unit(q, eps), rms_unit(k, eps)
    q = q * query_temperature(positions, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None, None]
    causal = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    out = torch.zeros(T, H, V, dtype=F)
    for head in range(H):
        g = head // (H // G)
        scores = (q[:, head] @ k[:, g].T) * m["scale"]
        out[:, head] = softmax_plus_one(scores, causal) @ v[:, g]
    gate = torch.sigmoid(h @ w[p + "g"].T)
    return (out.reshape(T, H * V) * gate) @ w[p + "o"].T


# ---- retention ---------------------------------------------------------------------------------------------------
def rotate_half(x, positions, base, dims):
    """x [T, heads, dim]: entry i of the first `dims` is paired with entry i + dims/2; the pair turns by p base^(-2i/dims)."""
    if dims == 0:
        return x
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    ang = positions.to(F)[:, None] * f[None, :]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    y = x.clone()
    y[..., :half] = a * c - b * s
    y[..., half:dims] = b * c + a * s
    return y


def decayed_recurrence(q, k, v, decay, gain=None):
    """Token by token: S <- decay_t S + gain_t k_t v_t^T, o_t = S^T q_t. q, k [T, N], v [T, P], decay and gain [T]."""
    T, N = q.shape
    S = torch.zeros(N, v.shape[1], dtype=F)
    out = torch.zeros(T, v.shape[1], dtype=F)
    for t in range(T):
        S = decay[t] * S + (1.0 if gain is None else gain[t]) * torch.outer(k[t], v[t])
        out[t] = S.T @ q[t]
    return out


def retention(h, w, p, m, eps, positions):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, D)
    k = (h @ w[p + "k"].T).view(T, H, D)
    v = (h @ w[p + "v"].T).view(T, H, V)
    q = rotate_half(q, positions, m["rot"]["base"], m["rot"]["dims"])
    k = rotate_half(k, positions, m["rot"]["base"], m["rot"]["dims"]) * D ** -0.5
    out = torch.zeros(T, H, V, dtype=F)
    for head in range(H):
        out[:, head] = decayed_recurrence(q[:, head], k[:, head], v[:, head], torch.full((T,), m["decay"][head], dtype=F))
    out = rms_unit(out, eps).reshape(T, H * V)
    return (out * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


def parallel_mixer(h, w, p, m, eps, positions):
    return (m["left_scale"] * sink_attention(h, w, p + "left.", m["left"], eps, positions)
            + m["right_scale"] * retention(h, w, p + "right.", m["right"], eps, positions))


# ---- state-space mixer -------------------------------------------------------------------------------------------
def causal_conv(x, taps, bias):
    """x [T, C], taps [C, K] (the last column is the current token's), zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=F), x], dim=0)
    out = bias.expand(T, C).clone()
    for j in range(K):
        out = out + padded[j:j + T] * taps[:, j]
    return out


def state_space_mixer(h, w, p, m, eps, positions=None):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w[p + "dt_bias"])
    decay = torch.exp(-torch.exp(w[p + "A_log"]) * dt)
    y = torch.zeros(T, H, P, dtype=F)
    for head in range(H):
        g = head // (H // G)
        y[:, head] = decayed_recurrence(C[:, g], B[:, g], x[:, head], decay[:, head], dt[:, head]) + w[p + "D"][head] * x[:, head]
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms_unit(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w[p + "norm"]
    return y @ w[p + "o"].T


# ---- feed-forward ------------------------------------------------------------------------------------------------
def expert(h, w, p):
    return gelu_erf(h @ w[p + "up"].T) @ w[p + "down"].T


def route(h, router, top):
    """(indices [T, top], weights [T, top]): the largest softmax scores, divided by their sum."""
    s = torch.softmax(h @ router.T, dim=-1)
    val, idx = torch.topk(s, top, dim=-1)
    return idx, val / (val.sum(-1, keepdim=True) + 1e-20)


def routed_feed_forward(h, w, p, f):
    idx, share = route(h, w[p + "router"], f["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for c in range(idx.shape[1]):
            out[t] += share[t, c] * expert(h[t:t + 1], w, f"{p}e{int(idx[t, c])}.")[0]
    if f.get("shared"):
        out = out + expert(h, w, p + "shared.")
    return out


# ---- the residual streams ----------------------------------------------------------------------------------------
def streams_read(xs, w_in):
    """xs [S, T, width] -> sum_s in[s] x_s."""
    return torch.einsum("s,stw->tw", w_in, xs)


def streams_write(xs, y, mix, w_out):
    """All streams at once from the old ones: x_t = sum_s mix[s, t] x_s + out[t] y."""
    return torch.einsum("sr,stw->rtw", mix, xs) + w_out[:, None, None] * y[None]


# ---- the whole model ---------------------------------------------------------------------------------------------
def forward(cfg, w, tokens, return_layers=False):
    """Logits [T, vocab] for one sequence from position 0; with return_layers also the sum of the streams after every layer."""
    eps = cfg["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    T = tokens.numel()
    positions = torch.arange(T)
    S = cfg.get("streams")
    x = w["embed"][tokens]
    xs = x[None].repeat(S, 1, 1) if S else None
    seen = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        mixer = parallel_mixer if layer["type"] == "parallel" else state_space_mixer
        subs = [(1, lambda u: mixer(u, w, p + "mix.", layer["mixer"], eps, positions))]
        if layer.get("mlp"):
            subs.append((2, lambda u: routed_feed_forward(u, w, p + "mlp.", layer["mlp"])))
        for q, sub in subs:
            norm = lambda u: layer_norm(u, w[f"{p}norm{q}"], w[f"{p}norm{q}.b"], eps)
            if S:
                y = sub(norm(streams_read(xs, w[f"{p}hc{q}.in"])))
                xs = streams_write(xs, y, w[f"{p}hc{q}.mix"], w[f"{p}hc{q}.out"])
            else:
                x = x + sub(norm(x))
        seen.append(xs.sum(0) if S else x)
    x = seen[-1] if seen else (xs.sum(0) if S else x)
    logits = layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["embed"].T * cfg["logit_scale"]
    return (logits, torch.stack(seen)) if return_layers else logits


# ---- random models -----------------------------------------------------------------------------------------------
def tensor_shapes(cfg):
    """name -> shape of every tensor of a model, written out from the design."""
    W = cfg["width"]
    S = cfg.get("streams")
    t = {"embed": (cfg["vocab"], W), "final.norm": (W,), "final.norm.b": (W,)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        subs = [1] + ([2] if layer.get("mlp") else [])
        for q in subs:
            t[f"{p}norm{q}"] = (W,)
            t[f"{p}norm{q}.b"] = (W,)
            if S:
                t[f"{p}hc{q}.in"] = (S,)
                t[f"{p}hc{q}.out"] = (S,)
                t[f"{p}hc{q}.mix"] = (S, S)
        if layer["type"] == "parallel":
            a, r = m["left"], m["right"]
            t[p + "mix.left.q"], t[p + "mix.left.q.b"] = (a["heads"] * a["dim"], W), (a["heads"] * a["dim"],)
            t[p + "mix.left.k"], t[p + "mix.left.k.b"] = (a["kv_heads"] * a["dim"], W), (a["kv_heads"] * a["dim"],)
            t[p + "mix.left.v"], t[p + "mix.left.v.b"] = (a["kv_heads"] * a["vdim"], W), (a["kv_heads"] * a["vdim"],)
            t[p + "mix.left.g"], t[p + "mix.left.o"] = (a["heads"] * a["vdim"], W), (W, a["heads"] * a["vdim"])
            t[p + "mix.right.q"] = t[p + "mix.right.k"] = (r["heads"] * r["dim"], W)
            t[p + "mix.right.v"] = t[p + "mix.right.g"] = (r["heads"] * r["vdim"], W)
            t[p + "mix.right.o"] = (W, r["heads"] * r["vdim"])
        else:
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            t[p + "mix.in"] = (2 * inner + 2 * gn + m["heads"], W)
            t[p + "mix.conv"], t[p + "mix.conv.b"] = (inner + 2 * gn, m["conv"]), (inner + 2 * gn,)
            t[p + "mix.dt_bias"] = t[p + "mix.A_log"] = t[p + "mix.D"] = (m["heads"],)
            t[p + "mix.norm"], t[p + "mix.o"] = (inner,), (W, inner)
        f = layer.get("mlp")
        if f:
            for e in range(f["router"]["experts"]):
                t[f"{p}mlp.e{e}.up"], t[f"{p}mlp.e{e}.down"] = (f["expert"]["ff"], W), (W, f["expert"]["ff"])
            t[p + "mlp.router"] = (f["router"]["experts"], W)
            if f.get("shared"):
                t[p + "mlp.shared.up"], t[p + "mlp.shared.down"] = (f["shared"]["ff"], W), (W, f["shared"]["ff"])
    return t


def random_weights(cfg, seed, scale=1.0):
    """Random bfloat16-representable weights, name -> float64 tensor, sized so that every mechanism shows in the logits."""
    g = torch.Generator().manual_seed(seed)
    w = {}
    S = cfg.get("streams") or 1
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        if name.endswith(".b"):          # a norm's bias is small, a projection's or a convolution's is not
            of = name[:-2].rsplit(".", 1)[-1]
            x = (0.1 if of.startswith("norm") else 0.3) * torch.randn(shape, generator=g)
        elif "norm" in last:
            x = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif last == "mix" and ".hc" in name:
            x = torch.eye(S) * 0.8 + 0.2 / S + 0.05 * torch.randn(shape, generator=g)
        elif last == "in" and ".hc" in name:
            x = 1.0 / S + 0.1 * torch.randn(shape, generator=g)
        elif last == "out" and ".hc" in name:
            x = 0.7 + 0.2 * torch.randn(shape, generator=g)
        elif last == "A_log":
            x = torch.log(0.5 + 2.0 * torch.rand(shape, generator=g))
        elif last == "dt_bias":
            x = torch.randn(shape, generator=g) - 2.0
        elif last == "D":
            x = 1.0 + 0.3 * torch.randn(shape, generator=g)
        elif last == "conv":
            x = 0.5 * torch.randn(shape, generator=g)
        elif name == "embed":
            x = torch.randn(shape, generator=g)
        elif last == "router":
            x = 6.0 * torch.randn(shape, generator=g) / math.sqrt(shape[-1])      # decisive: few tokens between two experts
        else:
            x = scale * 1.5 * torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        w[name] = x.to(torch.bfloat16).to(F)
    return w
