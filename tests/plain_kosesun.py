"""A plain, slow Kosesun: every mechanism as one small function in 64-bit torch on the CPU,
written from the equations, reading the raw ``config.json`` keys and the checkpoint's tensor
names directly.  It shares no code with ``pagedserve_amd``; the tests compare the engine with
it.  A whole sequence is always computed from its first token: there is no cache here."""

import math

import torch

F64 = torch.float64


def rms_norm(x, weight=None, eps=1e-6, offset=0.0):
    """x / sqrt(mean(x^2) + eps) * (offset + weight), over the last axis."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * (weight + offset)


def rotate_pairs(x, positions, dims, base):
    """x: [T, heads, dim].  Dimension 2i is paired with 2i+1 for i < dims / 2; the pair (a, b)
    at position p becomes (a cos t - b sin t, b cos t + a sin t), t = p base^(-2i/dims)."""
    out = x.clone()
    for i in range(dims // 2):
        theta = positions.to(F64) * (base ** (-2.0 * i / dims))
        c, s = torch.cos(theta)[:, None], torch.sin(theta)[:, None]
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def causal_attention_with_sink(q, k, v, scale, sink=None):
    """q: [T, H, d], k: [T, G, d], v: [T, G, dv]; query head h uses key/value head h // (H / G).
    Token i sees tokens j <= i.  ``sink[h]`` joins the softmax's denominator as exp(sink[h]);
    it has no key and no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros((T, H, v.shape[2]), dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            scores = (k[: i + 1, g] @ q[i, h]) * scale
            top = scores.max() if sink is None else torch.maximum(scores.max(), sink[h])
            weights = torch.exp(scores - top)
            total = weights.sum() + (0.0 if sink is None else torch.exp(sink[h] - top))
            out[i, h] = (weights / total) @ v[: i + 1, g]
    return out


def decay_of(z, tau):
    """sigmoid(z)^(1 / tau)."""
    return torch.sigmoid(z) ** (1.0 / tau)


def gated_recurrence(q, k, v, alpha, state=None):
    """Per head: S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.
    q, k, alpha: [T, H, d]; v: [T, H, dv]; state: [H, d, dv] (zero when None).  Returns (o, S_T)."""
    T, H, d = q.shape
    S = torch.zeros((H, d, v.shape[2]), dtype=F64) if state is None else state.clone()
    o = torch.zeros((T, H, v.shape[2]), dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return o, S


def hyper_read(streams, weights):
    """u = sum_s in[s] x_s."""
    return sum(weights[s] * streams[s] for s in range(len(streams)))


def hyper_write(streams, y, mix, out):
    """x'_t = sum_s mix[s, t] x_s + out[t] y, every new copy from the old ones."""
    count = len(streams)
    return [sum(mix[s, t] * streams[s] for s in range(count)) + out[t] * y for t in range(count)]


def squared_relu_feed_forward(h, up, down):
    return (torch.relu(h @ up.T) ** 2) @ down.T


def softcap(logits, cap):
    return cap * torch.tanh(logits / cap)


# ------------------------------------------------------------------ the mixers
def attention_mixer(W, prefix, mixer, eps, h, positions, shared):
    """``shared`` carries the first value-mixing layer's values to the later ones."""
    T = h.shape[0]
    H, G, d, dv = mixer["heads"], mixer.get("kv_heads", mixer["heads"]), mixer["dim"], mixer.get("vdim", mixer["dim"])
    q = rms_norm(h @ W[prefix + "q"].T, W[prefix + "q.norm"], eps).view(T, H, d)
    k = rms_norm(h @ W[prefix + "k"].T, W[prefix + "k.norm"], eps).view(T, G, d)
    v = (h @ W[prefix + "v"].T).view(T, G, dv)
    rot = mixer.get("rot")
    if rot:
        q = rotate_pairs(q, positions, rot["dims"], rot["base"])
        k = rotate_pairs(k, positions, rot["dims"], rot["base"])
    if mixer.get("v_mix"):
        if "first_values" in shared:
            lam = W[prefix + "vmix"]
            v = (1 - lam) * v + lam * shared["first_values"]
        else:
            shared["first_values"] = v
    o = causal_attention_with_sink(q, k, v, mixer["scale"], W[prefix + "sink"])
    gate = torch.sigmoid(h @ W[prefix + "g"].T)              # [T, H]
    return (o * gate[:, :, None]).reshape(T, H * dv) @ W[prefix + "o"].T


def gla_mixer(W, prefix, mixer, eps, h):
    T = h.shape[0]
    H, d, dv = mixer["heads"], mixer["dim"], mixer["vdim"]
    q = (h @ W[prefix + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ W[prefix + "k"].T).view(T, H, d)
    v = (h @ W[prefix + "v"].T).view(T, H, dv)
    z = (h @ W[prefix + "a1"].T) @ W[prefix + "a2"].T + W[prefix + "a2.b"]
    o, _ = gated_recurrence(q, k, v, decay_of(z, mixer["tau"]).view(T, H, d))
    o = rms_norm(o, W[prefix + "norm"], eps)
    gate = h @ W[prefix + "g"].T
    return (o.reshape(T, H * dv) * gate * torch.sigmoid(gate)) @ W[prefix + "o"].T


# ------------------------------------------------------------------ the model
def forward(raw, tensors, tokens):
    """Logits ``[T, vocab]`` of the whole sequence, and the summed stream after every layer."""
    W = {name: tensor.to(F64) for name, tensor in tensors.items()}
    eps = raw["norm"]["eps"]
    positions = torch.arange(len(tokens))
    x = W["embed"][torch.tensor(tokens)] * raw.get("embedding", {}).get("scale", 1.0)
    copies = raw.get("streams", 0)
    streams = [x.clone() for _ in range(max(copies, 1))]
    shared, after = {}, []
    for i, layer in enumerate(raw["layers"]):
        l = f"l{i}."
        sublayers = [(1, "mix")] + ([(2, "mlp")] if layer.get("mlp") else [])
        for q, what in sublayers:
            u = hyper_read(streams, W[l + f"hc{q}.in"]) if copies else streams[0]
            n = rms_norm(u, W[l + f"norm{q}"], eps, offset=1.0)
            if what == "mlp":
                y = squared_relu_feed_forward(n, W[l + "mlp.up"], W[l + "mlp.down"])
            elif layer["type"] == "attention":
                y = attention_mixer(W, l + "mix.", layer["mixer"], eps, n, positions, shared)
            else:
                y = gla_mixer(W, l + "mix.", layer["mixer"], eps, n)
            if copies:
                streams = hyper_write(streams, y, W[l + f"hc{q}.mix"], W[l + f"hc{q}.out"])
            else:
                streams = [streams[0] + y]
        after.append(sum(streams))
    x = rms_norm(sum(streams), W["final.norm"], eps, offset=1.0)
    logits = x @ W["head"].T
    cap = raw.get("logit_softcap")
    return (softcap(logits, cap) if cap else logits), after


def greedy_generate(raw, tensors, prompt, count):
    tokens = list(prompt)
    for _ in range(count):
        logits, _ = forward(raw, tensors, tokens)
        tokens.append(int(torch.argmax(logits[-1])))
    return tokens[len(prompt):]


# ------------------------------------------------------------------ random checkpoints
def random_checkpoint(raw, seed, decay_rank=4, lively=True):
    """Checkpoint tensors for a raw configuration, every part mattering: sinks of either sign,
    decays spread over (0, 1), stream weights away from the identity, sharp attention."""
    g = torch.Generator().manual_seed(seed)

    def normal(shape, std=1.0):
        return torch.randn(shape, generator=g) * std

    def matrix(rows, columns, gain=1.0):
        return normal((rows, columns), gain / math.sqrt(columns))

    d = raw["width"]
    out = {"embed": normal((raw["vocab"], d), 0.3)}
    copies = raw.get("streams", 0)
    for i, layer in enumerate(raw["layers"]):
        l, m = f"l{i}.", f"l{i}.mix."
        mixer = layer["mixer"]
        out[l + "norm1"] = normal((d,), 0.2)
        if layer["type"] == "attention":
            H, G = mixer["heads"], mixer.get("kv_heads", mixer["heads"])
            dk, dv = mixer["dim"], mixer.get("vdim", mixer["dim"])
            out[m + "q"] = matrix(H * dk, d, 2.0 if lively else 1.0)
            out[m + "k"] = matrix(G * dk, d, 2.0 if lively else 1.0)
            out[m + "v"] = matrix(G * dv, d)
            out[m + "g"] = matrix(H, d, 2.0)
            out[m + "o"] = matrix(d, H * dv)
            out[m + "q.norm"] = 1.0 + normal((H * dk,), 0.3)
            out[m + "k.norm"] = 1.0 + normal((G * dk,), 0.3)
            out[m + "sink"] = normal((H,), 1.5)
            if mixer.get("v_mix"):
                out[m + "vmix"] = torch.rand((), generator=g) * 0.5 + 0.25
        else:
            H, dk, dv = mixer["heads"], mixer["dim"], mixer["vdim"]
            out[m + "q"] = matrix(H * dk, d, 2.0)
            out[m + "k"] = matrix(H * dk, d)
            out[m + "v"] = matrix(H * dv, d)
            out[m + "g"] = matrix(H * dv, d, 2.0)
            out[m + "a1"] = matrix(decay_rank, d)
            out[m + "a2"] = matrix(H * dk, decay_rank, 3.0)
            out[m + "a2.b"] = 1.0 + normal((H * dk,), 2.0)
            out[m + "norm"] = 1.0 + normal((dv,), 0.3)
            out[m + "o"] = matrix(d, H * dv)
        if layer.get("mlp"):
            out[l + "norm2"] = normal((d,), 0.2)
            out[l + "mlp.up"] = matrix(layer["mlp"]["ff"], d)
            out[l + "mlp.down"] = matrix(d, layer["mlp"]["ff"])
        if copies:
            for q in (1, 2) if layer.get("mlp") else (1,):
                out[l + f"hc{q}.in"] = 1.0 / copies + normal((copies,), 0.2)
                out[l + f"hc{q}.out"] = 1.0 + normal((copies,), 0.3)
                out[l + f"hc{q}.mix"] = torch.eye(copies) + normal((copies, copies), 0.2)
    out["final.norm"] = normal((d,), 0.2)
    out["head"] = matrix(raw["vocab"], d, 2.0)
    return out
