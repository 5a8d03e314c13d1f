"""A plain, slow Zetunex in float64 on the CPU, written from the design's equations: one function
per mechanism, loops over tokens where the design has a recurrence.  It shares no code with the
engine; the tests hold the engine's kernels and whole models against it.

Notation: ``x`` the stream ``[T, d]``, ``u = rms_norm(x) * w`` a layer's input, ``m`` the factor on
what a layer adds.  Matrices are stored ``[out, in]`` and applied as ``W u``.
"""

import math

import torch

F64 = torch.float64


def rms_norm(x, weight, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ------------------------------------------------------------------ lightning attention
def decayed_recurrence(q, k, v, decay, state=None):
    """``S_t = decay_h S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t`` per head.  q, k: ``[T, H, dk]``,
    v: ``[T, H, dv]``, decay: ``[H]``; returns (o ``[T, H, dv]``, the last state ``[H, dk, dv]``)."""
    tokens, heads, dk = q.shape
    dv = v.shape[2]
    state = torch.zeros((heads, dk, dv), dtype=F64) if state is None else state.clone()
    out = torch.zeros((tokens, heads, dv), dtype=F64)
    for t in range(tokens):
        for h in range(heads):
            state[h] = decay[h] * state[h] + torch.outer(k[t, h], v[t, h])
            out[t, h] = state[h].T @ q[t, h]
    return out, state


def lightning(u, w, prefix, mixer, eps):
    tokens = u.shape[0]
    heads, dk, dv = mixer["heads"], mixer["dim"], mixer["vdim"]
    q = silu(u @ w[prefix + "q"].T).view(tokens, heads, dk)
    k = silu(u @ w[prefix + "k"].T).view(tokens, heads, dk)
    v = silu(u @ w[prefix + "v"].T).view(tokens, heads, dv)
    o, _ = decayed_recurrence(q, k, v, torch.tensor(mixer["decay"], dtype=F64))
    o = rms_norm(o.reshape(tokens, heads * dv), w[prefix + "norm"], eps)
    return (o * torch.sigmoid(u @ w[prefix + "g"].T)) @ w[prefix + "o"].T


# ------------------------------------------------------------------ windowed attention
def windowed_attention(q, k, v, scale, window):
    """Softmax attention of position i over the positions j with ``0 <= i - j < window`` (all
    earlier ones when ``window`` is 0); query head h reads key/value head ``h // (H / G)``."""
    tokens, heads, _ = q.shape
    groups = k.shape[1]
    out = torch.zeros((tokens, heads, v.shape[2]), dtype=F64)
    for i in range(tokens):
        first = max(0, i - window + 1) if window > 0 else 0
        for h in range(heads):
            g = h // (heads // groups)
            scores = (k[first:i + 1, g] @ q[i, h]) * scale
            out[i, h] = torch.softmax(scores, 0) @ v[first:i + 1, g]
    return out


def attention_half(u, w, prefix, left):
    tokens = u.shape[0]
    heads, groups, dk, dv = left["heads"], left["kv_heads"], left["dim"], left["vdim"]
    q = (u @ w[prefix + "q"].T + w[prefix + "q.b"]).view(tokens, heads, dk)
    k = (u @ w[prefix + "k"].T + w[prefix + "k.b"]).view(tokens, groups, dk)
    v = (u @ w[prefix + "v"].T + w[prefix + "v.b"]).view(tokens, groups, dv)
    o = windowed_attention(q, k, v, left["scale"], left["mask"]["size"])
    return o.reshape(tokens, heads * dv) @ w[prefix + "o"].T


# ------------------------------------------------------------------ selective scan
def causal_conv(raw, weight, bias, before=None):
    """``y_t[c] = bias[c] + sum_j weight[c, j] raw_(t - taps + 1 + j)[c]``: the last column is the
    current token's; ``before``: the ``taps - 1`` inputs ahead of the first (zeros if None)."""
    tokens, channels = raw.shape
    taps = weight.shape[1]
    if before is None:
        before = torch.zeros((taps - 1, channels), dtype=F64)
    padded = torch.cat([before, raw])
    out = torch.zeros((tokens, channels), dtype=F64)
    for t in range(tokens):
        out[t] = bias + (padded[t:t + taps].T * weight).sum(-1)
    return out


def selective_recurrence(x, dt, a, b, c, skip, state=None):
    """``S[c, n] = exp(dt_c a[c, n]) S[c, n] + dt_c x_c b_n``, ``y_c = sum_n S[c, n] c_n + skip_c x_c``."""
    tokens, channels = x.shape
    state = torch.zeros_like(a) if state is None else state.clone()
    y = torch.zeros((tokens, channels), dtype=F64)
    for t in range(tokens):
        state = torch.exp(dt[t].unsqueeze(1) * a) * state + (dt[t] * x[t]).unsqueeze(1) * b[t].unsqueeze(0)
        y[t] = state @ c[t] + skip * x[t]
    return y, state


def scan_half(u, w, prefix, right):
    inner, states, rank = right["inner"], right["state"], right["dt_rank"]
    both = u @ w[prefix + "in"].T
    raw, z = both[:, :inner], both[:, inner:]
    x = silu(causal_conv(raw, w[prefix + "conv"], w[prefix + "conv.b"]))
    low = x @ w[prefix + "x"].T
    dt = softplus(low[:, :rank] @ w[prefix + "dt"].T + w[prefix + "dt.b"])
    y, _ = selective_recurrence(x, dt, -torch.exp(w[prefix + "A_log"]), low[:, rank:rank + states],
                                low[:, rank + states:], w[prefix + "D"])
    return (y * silu(z)) @ w[prefix + "o"].T


def parallel(u, w, prefix, mixer, eps):
    a = rms_norm(attention_half(u, w, prefix + "left.", mixer["left"]), w[prefix + "left.out"], eps)
    b = rms_norm(scan_half(u, w, prefix + "right.", mixer["right"]), w[prefix + "right.out"], eps)
    return 0.5 * (a + b)


# ------------------------------------------------------------------ feed-forwards
def gated(u, gate, up, down):
    return (silu(u @ gate.T) * (u @ up.T)) @ down.T


def route(logits, groups, keep, top, scale):
    """Per row: (chosen experts, their weights).  Softmax over all experts; a group's score is
    its best expert's; only the ``keep`` best groups are open; the ``top`` best open experts are
    chosen with weight ``score * scale``."""
    chosen, weights = [], []
    experts = logits.shape[1]
    size = experts // groups
    for row in torch.softmax(logits, -1):
        best = sorted(range(groups), key=lambda g: -float(row[g * size:(g + 1) * size].max()))[:keep]
        open_ = [e for e in range(experts) if e // size in best]
        picked = sorted(open_, key=lambda e: -float(row[e]))[:top]
        chosen.append(picked)
        weights.append([float(row[e]) * scale for e in picked])
    return chosen, weights


def mixture(u, w, prefix, mlp):
    router = mlp["router"]
    groups = router.get("groups") or {}
    count = groups.get("count", 1)
    chosen, weights = route(u @ w[prefix + "router"].T, count, groups.get("keep", count),
                            router["top"], router.get("scale", 1.0))
    out = torch.zeros_like(u)
    for t in range(u.shape[0]):
        for e, weight in zip(chosen[t], weights[t]):
            p = f"{prefix}e{e}."
            out[t] += weight * gated(u[t:t + 1], w[p + "gate"], w[p + "up"], w[p + "down"])[0]
    return out


def feed_forward(u, w, prefix, mlp):
    if mlp["kind"] == "dense":
        return gated(u, w[prefix + "gate"], w[prefix + "up"], w[prefix + "down"])
    return mixture(u, w, prefix, mlp)


# ------------------------------------------------------------------ the model
def run_order(raw):
    """(layer, pass that this call opens or None) in the order in which the layers run."""
    count = len(raw["layers"])
    loop = raw.get("loop")
    if not loop:
        return [(i, None) for i in range(count)]
    order = [(i, None) for i in range(loop["start"])]
    for turn in range(loop["times"]):
        for i in range(loop["start"], loop["stop"]):
            order.append((i, turn if i == loop["start"] else None))
    return order + [(i, None) for i in range(loop["stop"], count)]


def forward(raw, tensors, tokens):
    """(logits ``[T, vocab]``, the stream after every layer run) of one sequence from its start."""
    w = {name: tensor.to(F64) for name, tensor in tensors.items()}
    eps = raw["norm"]["eps"]
    m = raw.get("residual_mult", 1.0)
    x = w["embed"][torch.tensor(list(tokens))]
    after = []
    for index, turn in run_order(raw):
        if turn is not None:
            x = x + w["loop.step"][turn]
        layer, prefix = raw["layers"][index], f"l{index}."
        u = rms_norm(x, w[prefix + "norm1"], eps)
        if layer["type"] == "lightning":
            y = lightning(u, w, prefix + "mix.", layer["mixer"], eps)
        else:
            y = parallel(u, w, prefix + "mix.", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            y = y + feed_forward(u, w, prefix + "mlp.", layer["mlp"])
        x = x + m * y
        after.append(x)
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T, after


def greedy_generate(raw, tensors, prompt, count):
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(int(forward(raw, tensors, tokens)[0][-1].argmax()))
    return tokens[len(prompt):]


# ------------------------------------------------------------------ random checkpoints
def random_checkpoint(raw, seed):
    """Checkpoint tensors (float32) of a random model of the raw configuration: matrices
    N(0, 1/in), scales around one, step sizes between 0.001 and 0.1."""
    g = torch.Generator().manual_seed(seed)

    def normal(*shape, std=1.0):
        return torch.randn(shape, generator=g) * std

    def matrix(rows, columns, gain=1.0):
        return normal(rows, columns, std=gain / math.sqrt(columns))

    d = raw["width"]
    w = {"embed": normal(raw["vocab"], d), "final.norm": 1 + normal(d, std=0.1)}
    if raw.get("loop"):
        w["loop.step"] = normal(raw["loop"]["times"], d, std=0.3)
    for i, layer in enumerate(raw["layers"]):
        p = f"l{i}."
        w[p + "norm1"] = 1 + normal(d, std=0.1)
        mixer = layer["mixer"]
        if layer["type"] == "lightning":
            heads, dk, dv = mixer["heads"], mixer["dim"], mixer["vdim"]
            for name, rows in (("q", heads * dk), ("k", heads * dk), ("v", heads * dv), ("g", heads * dv)):
                w[p + "mix." + name] = matrix(rows, d)
            w[p + "mix.o"] = matrix(d, heads * dv)
            w[p + "mix.norm"] = 1 + normal(heads * dv, std=0.1)
        else:
            left, right = mixer["left"], mixer["right"]
            a, s = p + "mix.left.", p + "mix.right."
            for name, rows in (("q", left["heads"] * left["dim"]), ("k", left["kv_heads"] * left["dim"]),
                               ("v", left["kv_heads"] * left["vdim"])):
                w[a + name] = matrix(rows, d)
                w[a + name + ".b"] = normal(rows, std=0.2)
            w[a + "o"] = matrix(d, left["heads"] * left["vdim"])
            w[a + "out"] = 1 + normal(d, std=0.1)
            inner, states, rank, taps = right["inner"], right["state"], right["dt_rank"], right["conv"]
            w[s + "in"] = matrix(2 * inner, d)
            w[s + "conv"] = normal(inner, taps, std=1 / math.sqrt(taps))
            w[s + "conv.b"] = normal(inner, std=0.1)
            w[s + "x"] = matrix(rank + 2 * states, inner)
            w[s + "dt"] = matrix(inner, rank)
            steps = torch.exp(torch.rand(inner, generator=g) * math.log(100.0) + math.log(1e-3))
            w[s + "dt.b"] = steps + torch.log(-torch.expm1(-steps))
            w[s + "A_log"] = torch.log(torch.arange(1, states + 1).float()).repeat(inner, 1) + normal(inner, states, std=0.1)
            w[s + "D"] = 1 + normal(inner, std=0.1)
            w[s + "o"] = matrix(d, inner)
            w[s + "out"] = 1 + normal(d, std=0.1)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        f = p + "mlp."
        if mlp["kind"] == "dense":
            w[f + "gate"], w[f + "up"], w[f + "down"] = matrix(mlp["ff"], d), matrix(mlp["ff"], d), matrix(d, mlp["ff"])
        else:
            # (logits a few units apart, so that no choice is a close call)
            w[f + "router"] = matrix(mlp["router"]["experts"], d, gain=3.0)
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                w[f + f"e{e}.gate"], w[f + f"e{e}.up"] = matrix(ff, d), matrix(ff, d)
                w[f + f"e{e}.down"] = matrix(d, ff)
    return w
