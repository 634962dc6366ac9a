"""Plain float64 oracle of the Tarulix design: one function per mechanism, whole
sequences at once, no caches, no batching. It shares no code with the library;
the library's serving path is compared against it.

Notation: a sequence of ``T`` tokens, residual ``x`` [T, W]; a linear map stored
``[out, in]`` is applied as ``x @ W.T``.
"""

import math

import torch

F64 = torch.float64


def f64(t):
    return t.to(F64)


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    """RMS norm whose weight is one number for all coordinates."""
    return unit_rms(x, eps) * float(g)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def distance_bucket(n: int, rows: int, far: float) -> int:
    """Row of the distance table for distance n >= 0: exact below rows/2, logarithmic up to ``far``, then the last."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def rotate_half_layout(x, positions, dims: int, base: float):
    """x [T, heads, D]: channel i < dims/2 pairs with channel i + dims/2; channels from ``dims`` on pass."""
    out = x.clone()
    half = dims // 2
    for i in range(half):
        f = base ** (-2.0 * i / dims)
        a = positions.to(F64) * f
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[:, :, i], x[:, :, i + half]
        out[:, :, i] = u * c - v * s
        out[:, :, i + half] = v * c + u * s
    return out


def biased_window_attention(h, p, c, eps, v_first=None):
    """Mixer 'attention': unit-RMS q/k, score * scale + table[bucket(i - j), head], window, softmax with a learned
    sink in the denominator, value mixing with the first such layer's values. ``p`` maps short names to tensors.
    Returns (output [T, W], the values that are cached [T, G, Dv])."""
    T = h.shape[0]
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = (h @ f64(p["q"]).T + f64(p["q.b"])).view(T, H, D)
    k = (h @ f64(p["k"]).T + f64(p["k.b"])).view(T, G, D)
    v = (h @ f64(p["v"]).T + f64(p["v.b"])).view(T, G, Dv)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    if c.get("v_mix") and v_first is not None:
        lam = float(p["vmix"])
        v = (1.0 - lam) * v + lam * v_first
    rel, sink = f64(p["rel"]), f64(p["sink"])
    rows, far, win = rel.shape[0], c["bias_max"], c["mask"]["size"]
    out = torch.zeros(T, H, Dv, dtype=F64)
    for i in range(T):
        js = [j for j in range(i + 1) if i - j < win]
        rows_of = torch.tensor([distance_bucket(i - j, rows, far) for j in js])
        for hh in range(H):
            g = hh // (H // G)
            s = (k[js, g] @ q[i, hh]) * c["scale"] + rel[rows_of, hh]
            m = torch.maximum(s.max(), sink[hh])
            e = torch.exp(s - m)
            w = e / (e.sum() + torch.exp(sink[hh] - m))
            out[i, hh] = w @ v[js, g]
    return out.reshape(T, H * Dv) @ f64(p["o"]).T + f64(p["o.b"]), v


def pooled_window_attention(h, p, c, eps):
    """Left half of mixer 'parallel': partial rotary (rotate-half layout), unit-RMS q/k after it, soft-capped score,
    window plus one mean key/value per block of ``pool`` tokens that lies wholly before the window, plain softmax,
    the heads' weights mixed by ``talk`` before they meet the values of each head's own kv head."""
    T = h.shape[0]
    H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    pos = torch.arange(T)
    q = (h @ f64(p["q"]).T + f64(p["q.b"])).view(T, H, D)
    k = (h @ f64(p["k"]).T + f64(p["k.b"])).view(T, G, D)
    v = (h @ f64(p["v"]).T + f64(p["v.b"])).view(T, G, Dv)
    q = unit_rms(rotate_half_layout(q, pos, c["rot"]["dims"], c["rot"]["base"]), eps)
    k = unit_rms(rotate_half_layout(k, pos, c["rot"]["dims"], c["rot"]["base"]), eps)
    win, P, cap = c["mask"]["size"], c["mask"]["pool"], c["softcap"]
    talk = f64(p["talk"])
    out = torch.zeros(T, H, Dv, dtype=F64)
    for i in range(T):
        blocks = [b for b in range(T // P + 1) if b * P + P - 1 <= i - win]
        js = [j for j in range(i + 1) if i - j < win]
        keys = [k[b * P:(b + 1) * P].mean(0) for b in blocks] + [k[j] for j in js]     # [n][G, D]
        vals = [v[b * P:(b + 1) * P].mean(0) for b in blocks] + [v[j] for j in js]
        K, V = torch.stack(keys), torch.stack(vals)
        w = torch.zeros(H, K.shape[0], dtype=F64)
        for hh in range(H):
            s = (K[:, hh // (H // G)] * q[i, hh]).sum(-1) * c["scale"]
            w[hh] = torch.softmax(cap * torch.tanh(s / cap), 0)
        w = talk @ w
        for hh in range(H):
            out[i, hh] = (w[hh][:, None] * V[:, hh // (H // G)]).sum(0)
    return out.reshape(T, H * Dv) @ f64(p["o"]).T + f64(p["o.b"])


def selective_scan_mixer(h, p, c):
    """Right half of mixer 'parallel': in-projection [x | z], causal per-channel convolution + silu on x,
    x-projection [dt | B | C], softplus step, S <- exp(dt A) S + dt x B, y = S C + D x, y * silu(z), out-projection."""
    T = h.shape[0]
    inner, N, R, taps = c["inner"], c["state"], c["dt_rank"], c["conv"]
    xz = h @ f64(p["in"]).T
    x, z = xz[:, :inner], xz[:, inner:]
    w, b = f64(p["conv"]), f64(p["conv.b"])
    padded = torch.cat([torch.zeros(taps - 1, inner, dtype=F64), x], 0)
    x = silu(sum(padded[j:j + T] * w[:, j] for j in range(taps)) + b)
    proj = x @ f64(p["x"]).T
    dt = torch.nn.functional.softplus(proj[:, :R] @ f64(p["dt"]).T + f64(p["dt.b"]), threshold=1e30)
    B, C = proj[:, R:R + N], proj[:, R + N:]
    A = -torch.exp(f64(p["A_log"]))
    S = torch.zeros(inner, N, dtype=F64)
    y = torch.zeros(T, inner, dtype=F64)
    for t in range(T):
        S = torch.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + f64(p["D"]) * x[t]
    return (y * silu(z)) @ f64(p["o"]).T


def gated_expert(h, p):
    return (silu(h @ f64(p["gate"]).T) * (h @ f64(p["up"]).T)) @ f64(p["down"]).T


def routed_mlp(h, p, c):
    """Softmax router over real + identity experts, choice by score + correction, weights = plain scores (not
    renormalised), identity experts return their input, a shared expert runs for every token."""
    E, I, top = c["router"]["experts"], c["router"].get("identity", 0), c["router"]["top"]
    s = torch.softmax(h @ f64(p["router"]).T, -1)                 # [T, E + I]
    choice = s + f64(p["correction"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in torch.topk(choice[t], top).indices.tolist():
            if e >= E:
                out[t] += s[t, e] * h[t]
            else:
                sub = {n: p[f"e{e}.{n}"] for n in ("gate", "up", "down")}
                out[t] += s[t, e] * gated_expert(h[t:t + 1], sub)[0]
    if c.get("shared"):
        out = out + gated_expert(h, {n: p[f"shared.{n}"] for n in ("gate", "up", "down")})
    return out


def sub(tensors, prefix):
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def model_forward(config, tensors, tokens):
    """tokens: list of ints. Returns (logits [T, vocab], [residual after each layer]) in float64."""
    eps = config["norm"]["eps"]
    x = f64(tensors["embed"])[torch.tensor(tokens)]
    v_first, residuals = None, []
    for i, spec in enumerate(config["layers"]):
        pre = f"l{i}."
        m = spec["mixer"]
        if spec["type"] == "attention":
            first = v_first if m.get("v_mix") else None
            y, v = biased_window_attention(x, sub(tensors, pre + "mix."), m, eps, first)
            if m.get("v_mix") and v_first is None:
                v_first = v
        elif spec["type"] == "parallel":
            y = m["left_scale"] * pooled_window_attention(x, sub(tensors, pre + "mix.left."), m["left"], eps) \
                + m["right_scale"] * selective_scan_mixer(x, sub(tensors, pre + "mix.right."), m["right"])
        else:
            raise ValueError(spec["type"])
        x = x + scalar_norm(y, tensors[pre + "norm1"], eps)
        if spec.get("mlp") is not None:
            x = x + scalar_norm(routed_mlp(x, sub(tensors, pre + "mlp."), spec["mlp"]), tensors[pre + "norm2"], eps)
        residuals.append(x.clone())
    x = scalar_norm(x, tensors["final.norm"], eps)
    return x @ f64(tensors["head"]).T, residuals


def forward(config, tensors, tokens):
    return model_forward(config, tensors, tokens)[0]


def random_checkpoint(config, seed=0, rel_rows=10):
    """Random tensors for a config, named and shaped as a checkpoint holds them (bfloat16)."""
    g = torch.Generator().manual_seed(seed)
    W = config["width"]
    out = {}

    def put(name, *shape, std=1.0, mean=0.0):
        out[name] = (torch.randn(shape, generator=g) * std + mean).to(torch.bfloat16)

    def attention(pre, c, extra):
        H, G, D, Dv = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
        for n, rows in (("q", H * D), ("k", G * D), ("v", G * Dv)):
            put(pre + n, rows, W, std=W ** -0.5)
            put(pre + n + ".b", rows, std=0.3)
        put(pre + "o", W, H * Dv, std=(H * Dv) ** -0.5)
        put(pre + "o.b", W, std=0.3)
        extra(H)

    def expert(pre, ff):
        put(pre + "gate", ff, W, std=W ** -0.5)
        put(pre + "up", ff, W, std=W ** -0.5)
        put(pre + "down", W, ff, std=ff ** -0.5)

    put("embed", config["vocab"], W)
    put("head", config["vocab"], W, std=W ** -0.5)
    put("final.norm", std=0.1, mean=1.2)
    for i, spec in enumerate(config["layers"]):
        pre, m = f"l{i}.", spec["mixer"]
        put(pre + "norm1", std=0.1, mean=0.8)
        if spec["type"] == "attention":
            def extra(H, pre=pre):
                put(pre + "mix.rel", rel_rows, H)
                put(pre + "mix.sink", H)
                put(pre + "mix.vmix", std=0.05, mean=0.35)
            attention(pre + "mix.", m, extra)
        else:
            def extra(H, pre=pre):
                out[pre + "mix.left.talk"] = (torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)).to(torch.bfloat16)
            attention(pre + "mix.left.", m["left"], extra)
            r, q = m["right"], pre + "mix.right."
            put(q + "in", 2 * r["inner"], W, std=W ** -0.5)
            put(q + "conv", r["inner"], r["conv"], std=0.5)
            put(q + "conv.b", r["inner"], std=0.2)
            put(q + "x", r["dt_rank"] + 2 * r["state"], r["inner"], std=r["inner"] ** -0.5)
            put(q + "dt", r["inner"], r["dt_rank"], std=r["dt_rank"] ** -0.5)
            put(q + "dt.b", r["inner"], std=0.5)
            put(q + "A_log", r["inner"], r["state"], std=0.5)
            put(q + "D", r["inner"])
            put(q + "o", W, r["inner"], std=r["inner"] ** -0.5)
        f = spec.get("mlp")
        if f is not None:
            put(pre + "norm2", std=0.1, mean=0.9)
            E, I = f["router"]["experts"], f["router"].get("identity", 0)
            put(pre + "mlp.router", E + I, W, std=2.0 * W ** -0.5)
            put(pre + "mlp.correction", E + I, std=0.05)
            for e in range(E):
                expert(pre + f"mlp.e{e}.", f["expert"]["ff"])
            if f.get("shared"):
                expert(pre + "mlp.shared.", f["shared"]["ff"])
    return out
