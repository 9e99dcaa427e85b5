"""A plain, slow Verorax in float64 on the CPU: one function per mechanism, whole sequences at once, no cache.
It shares nothing with the engine; the tests compare the engine with it.

cfg is the parsed config.json (a dict), w a dict name -> float64 tensor.
"""
import math

import torch

F = torch.float64
UNIT_EPS = 1e-6                      # under the root of a unit key of the delta rule
DECAY_RATE = math.exp(-0.5)          # the decay of a channel is exp(-DECAY_RATE * sigmoid(.)): between 0.545 and 1


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, weight, eps):
    return rms_unit(x, eps) * weight


def silu(z):
    return z * torch.sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def token_shift(h, mix):
    """Every row moves towards the row before it (zeros before the first) by the share `mix` of each channel; the
    rows before are taken as they were."""
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (before - h) * mix


def rotate_halves(x, positions, rot):
    """x [T, heads, dim]: entry i of the first rot['dims'] pairs with entry i + dims/2; the pair turns by
    position * base^(-2i/dims). The other entries stay."""
    dims = rot["dims"]
    half = dims // 2
    f = torch.tensor([rot["base"] ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    ang = positions.to(F)[:, None] * f[None, :]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    y = x.clone()
    y[..., :half] = a * c - b * s
    y[..., half:dims] = b * c + a * s
    return y


def visible(T, size=None):
    """[T, T] bool: row i sees column j (j <= i, and with a window i - j < size)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    m = j <= i
    if size is not None:
        m = m & (i - j < size)
    return m


def softmax_rows(scores, mask):
    s = scores.masked_fill(~mask, float("-inf"))
    e = torch.exp(s - s.max(-1, keepdim=True).values)
    return e / e.sum(-1, keepdim=True)


def latent_attention(h, w, p, m, eps):
    """Queries through a normed latent; keys and values of all heads from one normed latent a token, plus one rotated
    key part that the heads share."""
    T = h.shape[0]
    H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = norm(h @ w[p + ".dq"].T, w[p + ".dq.norm"], eps)
    q = (cq @ w[p + ".uq"].T).view(T, H, dn + dr)
    qn, qr = q[..., :dn], rotate_halves(q[..., dn:], pos, m["rot"])
    down = h @ w[p + ".dkv"].T
    c = norm(down[:, :R], w[p + ".dkv.norm"], eps)
    kr = rotate_halves(down[:, None, R:], pos, m["rot"])[:, 0]
    kn = (c @ w[p + ".uk"].T).view(T, H, dn)
    v = (c @ w[p + ".uv"].T).view(T, H, dv)
    mask = visible(T)
    out = torch.zeros(T, H, dv, dtype=F)
    for hd in range(H):
        s = (qn[:, hd] @ kn[:, hd].T + qr[:, hd] @ kr.T) * m["scale"]
        out[:, hd] = softmax_rows(s, mask) @ v[:, hd]
    return out.reshape(T, H * dv) @ w[p + ".o"].T


def differential_attention(h, w, p, m, eps):
    """Two windowed softmax attentions a head over the same values; the second, times lambda, is taken off the first,
    and the difference is brought to unit root mean square a head and scaled by 1 - diff."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + ".q"].T + w[p + ".q.b"]).view(T, H, 2, D)
    k = (h @ w[p + ".k"].T + w[p + ".k.b"]).view(T, G, 2, D)
    v = (h @ w[p + ".v"].T + w[p + ".v.b"]).view(T, G, V)
    lam = (torch.exp((w[p + ".lq1"] * w[p + ".lk1"]).sum()) - torch.exp((w[p + ".lq2"] * w[p + ".lk2"]).sum())
           + m["diff"])
    mask = visible(T, m["mask"]["size"])
    out = torch.zeros(T, H, V, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        maps = [softmax_rows((q[:, hd, i] @ k[:, g, i].T) * m["scale"], mask) @ v[:, g] for i in (0, 1)]
        out[:, hd] = rms_unit(maps[0] - lam * maps[1], eps) * (1.0 - m["diff"])
    return out.reshape(T, H * V) @ w[p + ".o"].T


def gated_window_attention(h, w, p, m, eps):
    """The left half of 'parallel': per-head q/k norm, a rotation of part of each head, a temperature a head on the
    scores, a window, and one sigmoid gate a head on the output."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = norm((h @ w[p + ".q"].T).view(T, H, D), w[p + ".q.norm"], eps)
    k = norm((h @ w[p + ".k"].T).view(T, G, D), w[p + ".k.norm"], eps)
    v = (h @ w[p + ".v"].T).view(T, G, V)
    q, k = rotate_halves(q, pos, m["rot"]), rotate_halves(k, pos, m["rot"])
    gate = torch.sigmoid(h @ w[p + ".g"].T)                     # [T, H]
    mask = visible(T, m["mask"]["size"])
    out = torch.zeros(T, H, V, dtype=F)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"] * w[p + ".temp"][hd]
        out[:, hd] = (softmax_rows(s, mask) @ v[:, g]) * gate[:, hd:hd + 1]
    return out.reshape(T, H * V) @ w[p + ".o"].T


def decayed_delta_rule(h, w, p, m, eps):
    """The right half of 'parallel': a state S [dim, dim] a head; every token each key channel decays by its own
    factor, a share of what the state holds along the unit key is removed, and k v^T is written."""
    T = h.shape[0]
    H, D = m["heads"], m["dim"]
    r = (h @ w[p + ".r"].T).view(T, H, D)
    k = (h @ w[p + ".k"].T).view(T, H, D)
    v = (h @ w[p + ".v"].T).view(T, H, D)
    decay = torch.exp(-DECAY_RATE * torch.sigmoid(torch.tanh(h @ w[p + ".w1"].T) @ w[p + ".w2"].T + w[p + ".w0"])).view(T, H, D)
    a = torch.sigmoid(h @ w[p + ".a"].T + w[p + ".a.b"]).view(T, H, D)
    u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + UNIT_EPS)
    o = torch.zeros(T, H, D, dtype=F)
    for hd in range(H):
        S = torch.zeros(D, D, dtype=F)
        for t in range(T):
            held = u[t, hd] @ S                                  # what the old state answers to the unit key
            S = decay[t, hd][:, None] * S - torch.outer(a[t, hd] * u[t, hd], held) + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ r[t, hd]
    o = rms_unit(o, eps).reshape(T, H * D) * w[p + ".norm"] * torch.sigmoid(h @ w[p + ".g"].T)
    return o @ w[p + ".o"].T


def parallel(h, w, p, m, eps):
    return (m["left_scale"] * gated_window_attention(h, w, p + ".left", m["left"], eps)
            + m["right_scale"] * decayed_delta_rule(h, w, p + ".right", m["right"], eps))


def dense_ff(h, w, p):
    return (gelu_tanh(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


CLOSE_CALL = 0.05     # choice scores nearer than this may fall either way once the router's input is rounded


def chosen_experts(h, w, p, f, given=None):
    """(indices [T, top], weights [T, top]): softmax over all router outputs; the correction only moves the choice.
    given {row: [experts]}: the choice somebody else made for some rows (an engine whose router read rounded rows). It
    is taken over where it could be right: every expert it names scores within CLOSE_CALL of the last one chosen here,
    and every expert chosen here that it leaves out is within CLOSE_CALL of the best one it could have left out."""
    top = f["router"]["top"]
    s = torch.softmax(h @ w[p + ".router"].T, dim=-1)
    choice = s + w[p + ".correction"]
    idx = torch.topk(choice, top, dim=-1).indices
    for t, other in (given or {}).items():
        assert len(other) == top == len(set(other)), f"{p} row {t}: {other} are not {top} experts"
        line = choice[t, idx[t]].min().item()
        assert all(choice[t, e].item() > line - CLOSE_CALL for e in other), f"{p} row {t}: {other} chosen, {idx[t].tolist()} score best"
        assert all(choice[t, e].item() < line + CLOSE_CALL for e in idx[t].tolist() if e not in other), \
            f"{p} row {t}: {other} chosen, {idx[t].tolist()} score best"
        idx[t] = torch.tensor(other)
    return idx, torch.gather(s, 1, idx)


def routed_ff(h, w, p, f, given=None):
    E = f["router"]["experts"]
    idx, share = chosen_experts(h, w, p, f, given)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, s in zip(idx[t].tolist(), share[t]):
            if e >= E:                                           # an identity expert hands the input on
                out[t] += s * h[t]
            else:
                x = h[t]
                out[t] += s * ((silu(w[f"{p}.e{e}.gate"] @ x) * (w[f"{p}.e{e}.up"] @ x)) @ w[f"{p}.e{e}.down"].T)
    return out


MIXERS = {"latent_attention": latent_attention, "attention": differential_attention, "parallel": parallel}


def layer(x, w, cfg, i, given=None):
    """One entry of the layer list on the stream x [T, width]; an entry with weights_of reads that layer's tensors.
    given: see chosen_experts."""
    l = cfg["layers"][i]
    p = f"l{l.get('weights_of', i)}"
    eps = cfg["norm"]["eps"]
    h = token_shift(norm(x, w[p + ".norm1"], eps), w[p + ".shift"])
    x = x + norm(MIXERS[l["type"]](h, w, p + ".mix", l["mixer"], eps), w[p + ".norm1b"], eps)
    f = l.get("mlp")
    if f is not None:
        h = norm(x, w[p + ".norm2"], eps)
        y = dense_ff(h, w, p + ".mlp") if f["kind"] == "dense" else routed_ff(h, w, p + ".mlp", f, given)
        x = x + norm(y, w[p + ".norm2b"], eps)
    return x


def forward(tokens, w, cfg, streams=None, choices=None):
    """Logits [T, vocab] of a whole sequence; `streams`, a list, receives the stream after every layer.
    choices {(layer, row): [experts]}: routing choices to take over where they could be right (chosen_experts)."""
    x = w["embed"][torch.as_tensor(tokens)]
    for i in range(len(cfg["layers"])):
        x = layer(x, w, cfg, i, {t: e for (l, t), e in (choices or {}).items() if l == i})
        if streams is not None:
            streams.append(x)
    return norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["head"].T


# ---- made-up weights for the tests -------------------------------------------------------------------------------
def tensor_shapes(cfg, low=6):
    """name -> shape of every tensor a configuration asks for; `low`: the inner size of the decay projections (the
    configuration does not hold it: the engine reads it off the tensor)."""
    W, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"]), "final.norm": (cfg["width"],), "head": (cfg["vocab"], cfg["width"])}
    for i, l in enumerate(cfg["layers"]):
        if "weights_of" in l:
            continue
        p, m = f"l{i}", l["mixer"]
        for n in ("norm1", "norm1b", "shift"):
            out[f"{p}.{n}"] = (W,)
        if l["type"] == "latent_attention":
            H, dn, dr, dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out.update({f"{p}.mix.dq": (Q, W), f"{p}.mix.dq.norm": (Q,), f"{p}.mix.uq": (H * (dn + dr), Q),
                        f"{p}.mix.dkv": (R + dr, W), f"{p}.mix.dkv.norm": (R,), f"{p}.mix.uk": (H * dn, R),
                        f"{p}.mix.uv": (H * dv, R), f"{p}.mix.o": (W, H * dv)})
        elif l["type"] == "attention":
            H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            out.update({f"{p}.mix.q": (2 * H * D, W), f"{p}.mix.q.b": (2 * H * D,), f"{p}.mix.k": (2 * G * D, W),
                        f"{p}.mix.k.b": (2 * G * D,), f"{p}.mix.v": (G * V, W), f"{p}.mix.v.b": (G * V,),
                        f"{p}.mix.o": (W, H * V)})
            for n in ("lq1", "lk1", "lq2", "lk2"):
                out[f"{p}.mix.{n}"] = (D,)
        else:
            a, r = m["left"], m["right"]
            H, G, D, V = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            out.update({f"{p}.mix.left.q": (H * D, W), f"{p}.mix.left.k": (G * D, W), f"{p}.mix.left.v": (G * V, W),
                        f"{p}.mix.left.q.norm": (D,), f"{p}.mix.left.k.norm": (D,), f"{p}.mix.left.temp": (H,),
                        f"{p}.mix.left.g": (H, W), f"{p}.mix.left.o": (W, H * V)})
            s = r["heads"] * r["dim"]
            rank = r.get("decay_rank", low)
            for n in ("r", "k", "v", "g", "a"):
                out[f"{p}.mix.right.{n}"] = (s, W)
            out.update({f"{p}.mix.right.a.b": (s,), f"{p}.mix.right.w1": (rank, W), f"{p}.mix.right.w2": (s, rank),
                        f"{p}.mix.right.w0": (s,), f"{p}.mix.right.norm": (s,), f"{p}.mix.right.o": (W, s)})
        f = l.get("mlp")
        if f is not None:
            out[f"{p}.norm2"] = out[f"{p}.norm2b"] = (W,)
            if f["kind"] == "dense":
                out.update({f"{p}.mlp.gate": (f["ff"], W), f"{p}.mlp.up": (f["ff"], W), f"{p}.mlp.down": (W, f["ff"])})
            else:
                E, n = f["router"]["experts"], f["router"]["experts"] + f["router"].get("identity", 0)
                out.update({f"{p}.mlp.router": (n, W), f"{p}.mlp.correction": (n,)})
                for e in range(E):
                    I = f["expert"]["ff"]
                    out.update({f"{p}.mlp.e{e}.gate": (I, W), f"{p}.mlp.e{e}.up": (I, W), f"{p}.mlp.e{e}.down": (W, I)})
    return out


def random_weights(cfg, seed, low=6):
    """bfloat16 tensors of sizes that keep every mechanism awake: products of unit spread, gains around one, shares
    between 0 and 1, router corrections large enough to change choices, decay and removal parameters spread over a
    few units."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, low).items():
        last = name.split(".")[-1]
        x = torch.randn(shape, generator=g)
        if name == "embed":
            t = x
        elif last == "shift":
            t = torch.rand(shape, generator=g)
        elif last in ("norm1", "norm1b", "norm2", "norm2b", "norm", "temp"):
            t = 1.0 + x * 0.2
        elif last == "correction":
            t = x * 0.1
        elif last == "router":
            t = x * (3.0 / shape[-1] ** 0.5)
        elif last in ("w0", "b"):
            t = x * 0.8
        elif last in ("lq1", "lk1", "lq2", "lk2"):
            t = x * 0.3
        elif last == "w2":
            t = x * (2.5 / shape[-1] ** 0.5)
        else:
            t = x * (1.5 / shape[-1] ** 0.5)
        out[name] = t.to(torch.bfloat16)
    return out


def as_float64(w):
    return {k: v.to(F) for k, v in w.items()}
