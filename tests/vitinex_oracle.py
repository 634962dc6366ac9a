"""A plain, slow float64 implementation of the Vitinex design, one function per
mechanism, written from the design's equations. It shares no code with
``colossalai_amd``: the tests compare the framework against it.

Notation: ``h`` is a sublayer's input ``[T, W]`` (one sequence, T tokens from
position 0), weights are ``[out, in]`` and applied as ``h @ W.T``; ``P`` is a
dict of the checkpoint's tensors by name.
"""

import math

import torch

F64 = torch.float64


def lin(h, w, b=None):
    y = h @ w.to(F64).T
    return y if b is None else y + b.to(F64)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w.to(F64)


def rotate_pairs(x, positions, base, dims):
    """x [T, ..., R]: pairs (2i, 2i+1), i < dims/2, turn by positions * base^(-2i/dims); the rest is kept."""
    out = x.clone()
    for i in range(dims // 2):
        ang = positions.to(F64) * (float(base) ** (-2.0 * i / dims))
        shape = [x.shape[0]] + [1] * (x.dim() - 2)
        c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def latent_attention_core(q, q_rot, lat, k_rot, w_uk, w_uv, scale, q_pos, k_pos):
    """q [T, H, D] plain and q_rot [T, H, R] rotated query parts; lat [S, rank] normed latents and k_rot [S, R] the
    rotated key part all heads share; w_uk [H * D, rank], w_uv [H * Dv, rank]. Head h's key is its slice of
    ``w_uk lat`` next to ``k_rot``, its value its slice of ``w_uv lat``; query i sees the keys j with
    k_pos[j] <= q_pos[i]. Returns [T, H, Dv]."""
    T, H, D = q.shape
    S = lat.shape[0]
    k_plain = lin(lat, w_uk).view(S, H, D)
    v = lin(lat, w_uv).view(S, H, -1)
    score = (torch.einsum("thd,shd->hts", q, k_plain) + torch.einsum("thr,sr->hts", q_rot, k_rot)) * scale
    seen = q_pos.view(-1, 1) >= k_pos.view(1, -1)
    score = score.masked_fill(~seen, float("-inf"))
    return torch.einsum("hts,shv->thv", torch.softmax(score, -1), v)


def latent_attention(h, P, pre, c, eps, positions=None):
    """Queries through a normed latent; keys and values up-projected from a normed latent; one rotated key part
    shared by all heads; causal softmax; per-head sigmoid output gate."""
    T = h.shape[0]
    H, D, R, Dv, rank = c["heads"], c["dim"], c["rot_dim"], c["vdim"], c["kv_rank"]
    pos = torch.arange(T) if positions is None else positions
    cq = rms_unit(lin(h, P[pre + "dq"]), eps) * P[pre + "dq.norm"].to(F64)
    q = lin(cq, P[pre + "uq"]).view(T, H, D + R)
    dkv = lin(h, P[pre + "dkv"])
    lat = rms_unit(dkv[:, :rank], eps) * P[pre + "dkv.norm"].to(F64)
    k_rot = rotate_pairs(dkv[:, rank:].clone(), pos, c["rot"]["base"], c["rot"]["dims"])     # [T, R]
    q_rot = rotate_pairs(q[..., D:].clone(), pos, c["rot"]["base"], c["rot"]["dims"])        # [T, H, R]
    o = latent_attention_core(q[..., :D], q_rot, lat, k_rot, P[pre + "uk"], P[pre + "uv"], c["scale"], pos, pos)
    o = o * torch.sigmoid(lin(h, P[pre + "g"]))[:, :, None]
    return lin(o.reshape(T, H * Dv), P[pre + "o"])


def causal_conv(x, taps, bias, history=None):
    """x [T, C]; taps [C, K] with the last column on the current token; zeros (or ``history`` [K-1, C]) before."""
    K = taps.shape[1]
    past = torch.zeros(K - 1, x.shape[1], dtype=F64) if history is None else history
    full = torch.cat([past, x], 0)
    y = torch.zeros_like(x)
    for j in range(K):
        y = y + full[j : j + x.shape[0]] * taps.to(F64)[:, j]
    return y + bias.to(F64), full[full.shape[0] - (K - 1):]


def ssd_scan(x, B, C, dt, A_log, D_skip, groups, S0=None):
    """x [T, H, V], B/C [T, G, N], dt [T, H] (after softplus). Per head h (group h // (H / G)):
    S_t = exp(-exp(A_log_h) dt) S_(t-1) + dt B_t x_t^T (S is N x V); y_t = S_t^T C_t + D_h x_t. Token by token."""
    T, H, V = x.shape
    N = B.shape[2]
    S = torch.zeros(H, N, V, dtype=F64) if S0 is None else S0.clone()
    y = torch.zeros(T, H, V, dtype=F64)
    per = H // groups
    head_group = torch.arange(H) // per
    for t in range(T):
        Bt, Ct = B[t][head_group], C[t][head_group]                      # [H, N]
        decay = torch.exp(-torch.exp(A_log.to(F64)) * dt[t])             # [H]
        S = decay[:, None, None] * S + dt[t][:, None, None] * Bt[:, :, None] * x[t][:, None, :]
        y[t] = torch.einsum("hnv,hn->hv", S, Ct) + D_skip.to(F64)[:, None] * x[t]
    return y, S


def mamba2(h, P, pre, c, eps):
    T = h.shape[0]
    H, V, N, G = c["heads"], c["vdim"], c["state"], c["groups"]
    inner = H * V
    p = lin(h, P[pre + "in"])
    z, xbc, dt = p[:, :inner], p[:, inner : 2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    xbc, _ = causal_conv(xbc, P[pre + "conv"], P[pre + "conv.b"])
    xbc = silu(xbc)
    x = xbc[:, :inner].reshape(T, H, V)
    B = xbc[:, inner : inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + P[pre + "dt_bias"].to(F64))
    y, _ = ssd_scan(x, B, C, dt, P[pre + "A_log"].to(F64), P[pre + "D"].to(F64), G)
    y = y.reshape(T, inner) * silu(z)
    ng = c["norm_groups"]
    y = rms_unit(y.view(T, ng, inner // ng), eps).reshape(T, inner) * P[pre + "norm"].to(F64)
    return lin(y, P[pre + "o"])


def dense_ff(h, P, pre):
    g = lin(h, P[pre + "gate"], P[pre + "gate.b"])
    u = lin(h, P[pre + "up"], P[pre + "up.b"])
    return lin(gelu_tanh(g) * u, P[pre + "down"], P[pre + "down.b"])


def expert(h, P, pre):
    return lin(torch.relu(lin(h, P[pre + "up"])) ** 2, P[pre + "down"])


def route(h, w_router, top):
    """Softmax over all experts; the ``top`` largest scores are chosen and kept as they are."""
    s = torch.softmax(lin(h, w_router), -1)
    idx = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :top]
    return idx, s.gather(1, idx)


def moe_ff(h, P, pre, c):
    idx, w = route(h, P[pre + "router"], c["router"]["top"])
    out = torch.zeros(h.shape[0], P[pre + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            out[t] += w[t, j] * expert(h[t : t + 1], P, pre + "e%d." % int(idx[t, j]))[0]
    if c.get("shared"):
        out = out + expert(h, P, pre + "shared.") * torch.sigmoid(lin(h, P[pre + "shared.sg"]))
    return out


def layer_runs(cfg):
    """Which layer runs when: (layer, pass number or None, first of its pass)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["stop"] <= loop["start"]:
        return [(i, None, False) for i in range(n)]
    runs = [(i, None, False) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t, i == loop["start"]) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None, False) for i in range(loop["stop"], n)]


def forward(cfg, P, tokens, residuals=None):
    """tokens: list of ids of one sequence -> float64 logits [T, vocab]."""
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    x = P["embed"].to(F64)[torch.tensor(tokens)]
    x0 = x.clone()
    for i, t, first in layer_runs(cfg):
        spec, pre = cfg["layers"][i], "l%d." % i
        if first:
            x = lin(torch.cat([x, x0], -1), P["loop.in"]) + P["loop.step"].to(F64)[t]
        h = layer_norm(x, P[pre + "norm1"], eps)
        if spec["type"] == "latent_attention":
            y = latent_attention(h, P, pre + "mix.", spec["mixer"], eps)
        elif spec["type"] == "mamba2":
            y = mamba2(h, P, pre + "mix.", spec["mixer"], eps)
        else:
            raise ValueError(spec["type"])
        x = x + m * layer_norm(y, P[pre + "norm1b"], eps)
        if spec.get("mlp") is not None:
            h = layer_norm(x, P[pre + "norm2"], eps)
            y = dense_ff(h, P, pre + "mlp.") if spec["mlp"]["kind"] == "dense" else moe_ff(h, P, pre + "mlp.", spec["mlp"])
            x = x + m * layer_norm(y, P[pre + "norm2b"], eps)
        if residuals is not None:
            residuals.append(x.clone())
    return lin(layer_norm(x, P["final.norm"], eps), P["embed"])


# ------------------------------------------------------------------ random models
def random_checkpoint(cfg, seed=0, dtype=torch.bfloat16):
    """Random tensors of a config's shapes, rounded to ``dtype`` (what a checkpoint would hold)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    P = {}

    def mat(name, o, i, gain=1.0):
        P[name] = (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).to(dtype)

    def vec(name, n, mean=0.0, std=0.1):
        P[name] = (mean + std * torch.randn(n, generator=g)).to(dtype)

    mat("embed", cfg["vocab"], W, math.sqrt(W))
    vec("final.norm", W, 1.0)
    loop = cfg.get("loop")
    if loop:
        mat("loop.in", W, 2 * W)
        P["loop.step"] = (0.3 * torch.randn(loop["times"], W, generator=g)).to(dtype)
    for i, spec in enumerate(cfg["layers"]):
        p, c = "l%d." % i, spec["mixer"]
        for n in ("norm1", "norm1b"):
            vec(p + n, W, 1.0)
        if spec["type"] == "latent_attention":
            H, D, R, Dv = c["heads"], c["dim"], c["rot_dim"], c["vdim"]
            mat(p + "mix.dq", c["q_rank"], W)
            vec(p + "mix.dq.norm", c["q_rank"], 1.0)
            mat(p + "mix.uq", H * (D + R), c["q_rank"], 2.0)
            mat(p + "mix.dkv", c["kv_rank"] + R, W, 2.0)
            vec(p + "mix.dkv.norm", c["kv_rank"], 1.0)
            mat(p + "mix.uk", H * D, c["kv_rank"], 2.0)
            mat(p + "mix.uv", H * Dv, c["kv_rank"])
            mat(p + "mix.g", H, W)
            mat(p + "mix.o", W, H * Dv)
        else:
            H, V, N, G, K = c["heads"], c["vdim"], c["state"], c["groups"], c["conv"]
            inner, ch = H * V, H * V + 2 * G * N
            mat(p + "mix.in", 2 * inner + 2 * G * N + H, W)
            P[p + "mix.conv"] = (torch.randn(ch, K, generator=g) * 0.5).to(dtype)
            vec(p + "mix.conv.b", ch)
            vec(p + "mix.dt_bias", H, -1.0, 0.5)
            vec(p + "mix.A_log", H, -0.5, 0.5)
            vec(p + "mix.D", H, 1.0, 0.3)
            vec(p + "mix.norm", inner, 1.0)
            mat(p + "mix.o", W, inner)
        f = spec.get("mlp")
        if f is None:
            continue
        for n in ("norm2", "norm2b"):
            vec(p + n, W, 1.0)
        if f["kind"] == "dense":
            for n, o, i_ in (("gate", f["ff"], W), ("up", f["ff"], W), ("down", W, f["ff"])):
                mat(p + "mlp." + n, o, i_)
                vec(p + "mlp." + n + ".b", o)
        else:
            for e in range(f["router"]["experts"]):
                mat(p + "mlp.e%d.up" % e, f["expert"]["ff"], W)
                mat(p + "mlp.e%d.down" % e, W, f["expert"]["ff"])
            mat(p + "mlp.router", f["router"]["experts"], W, 3.0)
            if f.get("shared"):
                mat(p + "mlp.shared.up", f["shared"]["ff"], W)
                mat(p + "mlp.shared.down", W, f["shared"]["ff"])
                mat(p + "mlp.shared.sg", 1, W)
    return P
