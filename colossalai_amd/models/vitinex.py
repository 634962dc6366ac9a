"""Vitinex: a decoder-only language model of latent-attention and state-space
layers with a looped block, served from paged latents plus fixed-size state.

Every layer norms a sublayer's input *and* its output (centred norm with a
weight, no bias) and adds the output scaled by a constant ``m``:
``x += m * N_out(mixer(N_in(x)))``, then ``x += m * N_out'(ff(N_in'(x)))``, with
four norm weights per layer.
The residual ``x`` is float32. A checkpoint's ``layers`` list picks per layer

* mixer ``latent_attention`` — queries through an RMS-normed low-rank latent;
  keys and values are up-projections of one RMS-normed latent per token, plus
  one rotated key part that all heads share (rotation on neighbouring pairs);
  causal softmax; per-head sigmoid output gate. Only the latent and the
  rotated part are paged: attention runs in the latent space
  (``ops/latent_attention.py``).
* mixer ``mamba2`` — a state-space recurrence with one decay per head: one
  input projection ``[z | x | B | C | dt]``, a short causal convolution with
  bias and SiLU over ``x, B, C``, ``S <- a S + dt B x^T``, ``y = S^T C + D x``,
  then ``y * silu(z)``, a grouped RMS norm and the output projection.
* feed-forward ``dense`` — ``down(gelu_tanh(gate h) * up h)`` with biases — or
  ``moe`` — bias-free squared-ReLU experts behind a float32 softmax router
  whose ``top`` largest scores are the mixing weights as they are, plus an
  optional shared expert scaled by a per-token sigmoid.

``loop = {start, stop, times}`` runs layers ``start .. stop - 1`` ``times``
times in a row with the same weights; each pass keeps its own pages and state
(the cache plan below is per layer *run*). Ahead of every pass the stream is
mixed with the embedding output, ``x <- W_in [x; x0] + step[t]``.
The logits reuse the embedding table.

Serving goes through ``forward_ragged`` (a ragged step over paged latents and
state slots); ``forward`` runs whole sequences through the same path with
throw-away caches.
"""

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..ops.activation import gelu_tanh_mul, relu_squared
from ..ops.group_norm import add_layer_norm, gated_grouped_rms_norm, grouped_rms_norm, layer_norm
from ..ops.latent_attention import latent_attention, latent_kv_write
from ..ops.linear_recurrence import ssd_recurrence
from ..ops.pair_rotary import pair_frequencies
from ..ops.ragged import RaggedBatch
from ..ops.routed_experts import grouped_topk_route, routed_expert_ffn
from ..ops.short_conv import short_conv
from .packed import PackedLinear
from .registry import register_model

__all__ = ["VitinexConfig", "VitinexForCausalLM"]


@dataclass
class VitinexConfig:
    vocab: int
    width: int
    layers: List[dict]
    norm_eps: float = 1e-6
    residual_mult: float = 1.0
    loop: Optional[dict] = None  # {"start", "stop", "times"}

    @classmethod
    def from_dict(cls, d: dict) -> "VitinexConfig":
        loop = d.get("loop")
        if loop is not None:
            loop = {k: int(loop[k]) for k in ("start", "stop", "times")}
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=list(d["layers"]),
                   norm_eps=float(d["norm"]["eps"]), residual_mult=float(d.get("residual_mult", 1.0)), loop=loop)

    def to_dict(self) -> dict:
        d = {"architecture": "Vitinex", "layers": self.layers, "norm": {"eps": self.norm_eps},
             "residual_mult": self.residual_mult, "vocab": self.vocab, "width": self.width}
        if self.loop is not None:
            d["loop"] = dict(self.loop)
        return d

    def layer_runs(self):
        """The order in which layers run: ``(layer, pass number or None, first of its pass)``."""
        n = len(self.layers)
        lp = self.loop
        if lp is None or lp["stop"] <= lp["start"] or lp["times"] < 1:
            return [(i, None, False) for i in range(n)]
        if not 0 <= lp["start"] < lp["stop"] <= n:
            raise ValueError(f"loop {lp} does not fit {n} layers")
        runs = [(i, None, False) for i in range(lp["start"])]
        for t in range(lp["times"]):
            runs += [(i, t, i == lp["start"]) for i in range(lp["start"], lp["stop"])]
        return runs + [(i, None, False) for i in range(lp["stop"], n)]


def _vec(n, value=1.0):
    return nn.Parameter(torch.full((n,), value, dtype=torch.float32))


class VitinexLatentAttention(nn.Module):
    def __init__(self, width: int, c: dict, eps: float):
        super().__init__()
        self.eps = eps
        self.H, self.D, self.R, self.Dv = int(c["heads"]), int(c["dim"]), int(c["rot_dim"]), int(c["vdim"])
        self.rank, self.q_rank = int(c["kv_rank"]), int(c["q_rank"])
        self.scale = float(c["scale"])
        rot = c["rot"]
        self.rot_base, self.rot_dims = float(rot["base"]), int(rot["dims"])
        if self.rot_dims > self.R or self.rot_dims % 2:
            raise ValueError(f"{self.rot_dims} rotated channels do not fit a rotated part of {self.R}")
        self.in_proj = PackedLinear(width, {"dq": self.q_rank, "dkv": self.rank + self.R, "g": self.H})
        self.dq_norm, self.dkv_norm = _vec(self.q_rank), _vec(self.rank)
        self.uq = nn.Linear(self.q_rank, self.H * (self.D + self.R), bias=False)
        self.uk = nn.Parameter(torch.randn(self.H, self.D, self.rank) * self.rank ** -0.5)
        self.uv = nn.Parameter(torch.randn(self.H, self.Dv, self.rank) * self.rank ** -0.5)
        self.o = nn.Linear(self.H * self.Dv, width, bias=False)
        self.register_buffer("freqs", pair_frequencies(self.rot_base, self.rot_dims), persistent=False)

    def kv_shape(self):
        """One key head holding the latent and the shared rotated part; the values are a view of it."""
        return (1, self.rank + self.R, 0)

    def state_buffers(self):
        return None

    def forward(self, h, batch: RaggedBatch, pool, state):
        N = h.shape[0]
        p, _ = self.in_proj(h)
        latent_kv_write(p["dkv"], self.dkv_norm, self.eps, self.freqs, pool, batch)
        cq = grouped_rms_norm(p["dq"], self.dq_norm, 1, self.eps, None, h.dtype)
        q = self.uq(cq).view(N, self.H, self.D + self.R)
        o = latent_attention(q, self.uk, self.uv, pool, batch, self.scale, self.freqs, self.rank, p["g"])
        return self.o(o)


class VitinexMamba2(nn.Module):
    def __init__(self, width: int, c: dict, eps: float):
        super().__init__()
        self.eps = eps
        self.H, self.V, self.N, self.G = int(c["heads"]), int(c["vdim"]), int(c["state"]), int(c["groups"])
        self.K, self.norm_groups = int(c["conv"]), int(c["norm_groups"])
        if self.H % self.G:
            raise ValueError(f"{self.H} heads do not split into {self.G} groups")
        self.inner = self.H * self.V
        self.C = self.inner + 2 * self.G * self.N
        if self.inner % self.norm_groups:
            raise ValueError(f"{self.inner} channels do not split into {self.norm_groups} norm groups")
        self.in_proj = nn.Linear(width, 2 * self.inner + 2 * self.G * self.N + self.H, bias=False)
        self.conv = nn.Parameter(torch.randn(self.C, self.K, dtype=torch.float32) * 0.5)
        self.conv_b = _vec(self.C, 0.0)
        self.dt_bias, self.A_log, self.D_skip = _vec(self.H, 0.0), _vec(self.H, 0.0), _vec(self.H)
        self.norm = _vec(self.inner)
        self.o = nn.Linear(self.inner, width, bias=False)

    def kv_shape(self):
        return None

    def state_buffers(self):
        buf = {"S": (self.H, self.N, self.V)}
        if self.K > 1:
            buf["tail"] = (self.K - 1, self.C)
        return buf

    def forward(self, h, batch: RaggedBatch, pool, state):
        N, inner, GN = h.shape[0], self.inner, self.G * self.N
        y = self.in_proj(h)
        # the convolution feeds a recurrence: its activated output stays float32
        xbc = short_conv(y[:, inner : inner + self.C], self.conv, state.get("tail"), batch, True, torch.float32,
                         self.conv_b)
        o = ssd_recurrence(xbc[:, :inner].view(N, self.H, self.V), xbc[:, inner : inner + GN].view(N, self.G, self.N),
                           xbc[:, inner + GN:].view(N, self.G, self.N), y[:, inner + self.C:], self.A_log,
                           self.dt_bias, self.D_skip, state["S"], batch)
        g = gated_grouped_rms_norm(o.view(N, inner), y[:, :inner], self.norm, self.norm_groups, self.eps, h.dtype)
        return self.o(g)


class VitinexDenseMLP(nn.Module):
    def __init__(self, width: int, c: dict):
        super().__init__()
        ff = int(c["ff"])
        self.in_proj = PackedLinear(width, {"gate": ff, "up": ff}, bias=True)
        self.down = nn.Linear(ff, width, bias=True)

    def forward(self, h):
        _, y = self.in_proj(h)
        return self.down(gelu_tanh_mul(y))


class VitinexExpert(nn.Module):
    """down(relu(up h)^2), no biases."""

    def __init__(self, width: int, ff: int):
        super().__init__()
        self.up = nn.Linear(width, ff, bias=False)
        self.down = nn.Linear(ff, width, bias=False)

    def forward(self, h):
        return self.down(relu_squared(self.up(h)))


class VitinexMoE(nn.Module):
    def __init__(self, width: int, c: dict):
        super().__init__()
        r = c["router"]
        self.E, self.top = int(r["experts"]), int(r["top"])
        if not 0 < self.top <= self.E:
            raise ValueError(f"cannot choose {self.top} of {self.E} experts")
        ff = int(c["expert"]["ff"])
        self.shared = VitinexExpert(width, int(c["shared"]["ff"])) if c.get("shared") else None
        # float32 always; with a shared expert its last row is the shared expert's gate
        self.router = nn.Parameter(torch.randn(self.E + (1 if self.shared is not None else 0), width,
                                               dtype=torch.float32) * width ** -0.5)
        self.w_up = nn.Parameter(torch.randn(self.E, ff, width) * width ** -0.5)
        self.w_down = nn.Parameter(torch.randn(self.E, width, ff) * ff ** -0.5)

    def forward(self, h):
        logits = F.linear(h.float(), self.router)
        ids, weights = grouped_topk_route(logits[:, : self.E], None, self.top, score="softmax", renorm=False)
        base = gate = None
        if self.shared is not None:
            base, gate = self.shared(h), logits[:, self.E]
        return routed_expert_ffn(h, self.w_up, self.w_down, ids, weights, base, "relu_squared", gate)


MIXERS = {"latent_attention": VitinexLatentAttention, "mamba2": VitinexMamba2}
MLPS = {"dense": VitinexDenseMLP, "moe": VitinexMoE}


class VitinexLayer(nn.Module):
    def __init__(self, cfg: VitinexConfig, spec: dict):
        super().__init__()
        if spec["type"] not in MIXERS:
            raise ValueError(f"unknown mixer type {spec['type']!r}")
        self.kind = spec["type"]
        self.norm1, self.norm1b = _vec(cfg.width), _vec(cfg.width)
        self.mix = MIXERS[spec["type"]](cfg.width, spec["mixer"], cfg.norm_eps)
        m = spec.get("mlp")
        if m is not None and m.get("kind") not in MLPS:
            raise ValueError(f"unknown feed-forward kind {m.get('kind')!r}")
        self.mlp = MLPS[m["kind"]](cfg.width, m) if m is not None else None
        if self.mlp is not None:
            self.norm2, self.norm2b = _vec(cfg.width), _vec(cfg.width)


@register_model("Vitinex")
class VitinexForCausalLM(nn.Module):
    config_class = VitinexConfig
    serves_ragged = True  # the serving engines drive forward_ragged

    def __init__(self, cfg: VitinexConfig):
        super().__init__()
        self.config = cfg
        self.embed = nn.Embedding(cfg.vocab, cfg.width)
        self.layers = nn.ModuleList([VitinexLayer(cfg, s) for s in cfg.layers])
        self.final_norm = _vec(cfg.width)
        self.runs = cfg.layer_runs()
        self.looped = any(first for _, _, first in self.runs)
        if self.looped:
            # the mix of the stream with the embedding output is float32 in either serving type: it replaces the
            # residual stream itself
            self.loop_in = nn.Parameter(torch.randn(cfg.width, 2 * cfg.width, dtype=torch.float32) * (2 * cfg.width) ** -0.5)
            self.loop_step = nn.Parameter(torch.zeros(cfg.loop["times"], cfg.width, dtype=torch.float32))

    # ------------------------------------------------------------ cache plan
    def kv_layer_shapes(self):
        """Per layer *run* ``(kv_heads, key_dim, value_dim)`` or None: a looped layer has one entry per pass."""
        return [self.layers[i].mix.kv_shape() for i, _, _ in self.runs]

    def state_layer_buffers(self):
        """Per layer run ``{name: shape}`` of float32 state kept per sequence, or None."""
        return [self.layers[i].mix.state_buffers() for i, _, _ in self.runs]

    @property
    def act_dtype(self):
        return self.embed.weight.dtype

    # ---------------------------------------------------------------- serve
    def forward_ragged(self, tokens: torch.Tensor, batch: RaggedBatch, kv, state,
                       want: Optional[torch.Tensor] = None, residuals: Optional[list] = None) -> torch.Tensor:
        """tokens [N] (flat, sequence after sequence as ``batch`` says); ``kv`` a KVCacheManager and ``state`` a
        StateCacheManager laid out by ``kv_layer_shapes`` / ``state_layer_buffers``. Returns float32 logits of the
        rows ``want`` (indices into the flat token axis; all rows if None). ``residuals``, when a list, receives a
        copy of the float32 residual stream after every layer run."""
        cfg, act = self.config, self.act_dtype
        eps, m = cfg.norm_eps, cfg.residual_mult
        x = self.embed(tokens).float()
        x0 = x.clone() if self.looped else None
        h = None
        n_runs = len(self.runs)
        for r, (i, t, first) in enumerate(self.runs):
            layer = self.layers[i]
            if first:
                x = torch.addmm(self.loop_step[t], torch.cat([x, x0], -1), self.loop_in.t())
                h = None
            if h is None:
                h = layer_norm(x, layer.norm1, eps, act)
            y = layer.mix(h, batch, kv.k_pools[r], state.layers[r])
            follows = r + 1 < n_runs and not self.runs[r + 1][2]
            next_w = self.layers[self.runs[r + 1][0]].norm1 if follows else None
            if layer.mlp is not None:
                h = add_layer_norm(x, y, layer.norm1b, m, layer.norm2, eps, act)
                h = add_layer_norm(x, layer.mlp(h), layer.norm2b, m, next_w, eps, act)
            else:
                h = add_layer_norm(x, y, layer.norm1b, m, next_w, eps, act)
            if residuals is not None:
                residuals.append(x.clone())
        if want is not None:
            x = x.index_select(0, want)
        return F.linear(layer_norm(x, self.final_norm, eps, act), self.embed.weight).float()

    def forward(self, input_ids: torch.Tensor) -> torch.Tensor:
        """input_ids [B, S] -> logits [B, S, vocab] (float32), every sequence from position 0 with caches that
        live for this call only."""
        from ..inference.kv_cache import KVCacheManager
        from ..inference.state_cache import StateCacheManager

        B, S = input_ids.shape
        dev = input_ids.device
        page = 16
        pages = (S + page - 1) // page
        kv = KVCacheManager(len(self.runs), 0, 0, num_blocks=B * pages, block_size=page, device=dev,
                            dtype=self.act_dtype, layer_shapes=self.kv_layer_shapes())
        state = StateCacheManager(self.state_layer_buffers(), B, device=dev)
        tables = [list(range(b * pages, (b + 1) * pages)) for b in range(B)]
        batch = RaggedBatch.build([S] * B, [0] * B, list(range(B)), dev, tables, page)
        with torch.no_grad():
            return self.forward_ragged(input_ids.reshape(-1), batch, kv, state).view(B, S, -1)

    # -------------------------------------------------------------- weights
    def load_checkpoint_tensors(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Pack a checkpoint's tensors (``embed``, ``loop.in``, ``loop.step``, ``l<i>.norm{1,1b,2,2b}``,
        ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``) into this module's parameters. Every tensor must be used
        and every parameter filled."""
        used = set()

        def get(name):
            used.add(name)
            return tensors[name]

        def put(param, value):
            assert tuple(param.shape) == tuple(value.shape), (tuple(param.shape), tuple(value.shape))
            param.data.copy_(value.to(param.dtype))

        put(self.embed.weight, get("embed"))
        put(self.final_norm, get("final.norm"))
        if self.looped:
            put(self.loop_in, get("loop.in"))
            put(self.loop_step, get("loop.step"))
        else:
            used.update(n for n in ("loop.in", "loop.step") if n in tensors)  # a loop that never runs
        for i, layer in enumerate(self.layers):
            p, m = f"l{i}.", layer.mix
            put(layer.norm1, get(p + "norm1"))
            put(layer.norm1b, get(p + "norm1b"))
            a = p + "mix."
            if layer.kind == "latent_attention":
                put(m.in_proj.weight, torch.cat([get(a + part) for part in m.in_proj.parts], 0))
                put(m.dq_norm, get(a + "dq.norm"))
                put(m.dkv_norm, get(a + "dkv.norm"))
                put(m.uq.weight, get(a + "uq"))
                put(m.uk, get(a + "uk").view(m.H, m.D, m.rank))
                put(m.uv, get(a + "uv").view(m.H, m.Dv, m.rank))
                put(m.o.weight, get(a + "o"))
            else:
                put(m.in_proj.weight, get(a + "in"))
                put(m.conv, get(a + "conv"))
                put(m.conv_b, get(a + "conv.b"))
                put(m.dt_bias, get(a + "dt_bias"))
                put(m.A_log, get(a + "A_log"))
                put(m.D_skip, get(a + "D"))
                put(m.norm, get(a + "norm"))
                put(m.o.weight, get(a + "o"))
            f, b = layer.mlp, p + "mlp."
            if f is None:
                used.update(n for n in (p + "norm2", p + "norm2b") if n in tensors)
                continue
            put(layer.norm2, get(p + "norm2"))
            put(layer.norm2b, get(p + "norm2b"))
            if isinstance(f, VitinexDenseMLP):
                put(f.in_proj.weight, torch.cat([get(b + "gate"), get(b + "up")], 0))
                put(f.in_proj.bias, torch.cat([get(b + "gate.b"), get(b + "up.b")], 0))
                put(f.down.weight, get(b + "down"))
                put(f.down.bias, get(b + "down.b"))
            else:
                rows = [get(b + "router")]
                if f.shared is not None:
                    rows.append(get(b + "shared.sg").view(1, -1))
                    put(f.shared.up.weight, get(b + "shared.up"))
                    put(f.shared.down.weight, get(b + "shared.down"))
                put(f.router, torch.cat(rows, 0))
                put(f.w_up, torch.stack([get(b + f"e{e}.up") for e in range(f.E)], 0))
                put(f.w_down, torch.stack([get(b + f"e{e}.down") for e in range(f.E)], 0))
        missing = set(tensors) - used
        if missing:
            raise ValueError(f"checkpoint tensors without a place in the model: {sorted(missing)[:8]}")

    @classmethod
    def from_checkpoint(cls, config: dict, tensors: Dict[str, torch.Tensor], dtype=torch.bfloat16, device="cpu"):
        """Build from a parsed config.json and a name -> tensor mapping. Matrices and projection biases take
        ``dtype``; norm weights, the convolution, decays, the router and the loop's mix stay float32."""
        model = cls(VitinexConfig.from_dict(config))
        keep32 = {id(l.mlp.router) for l in model.layers if isinstance(l.mlp, VitinexMoE)}
        keep32 |= {id(l.mix.conv) for l in model.layers if l.kind == "mamba2"}
        if model.looped:
            keep32 |= {id(model.loop_in), id(model.loop_step)}
        for p in model.parameters():
            if p.dim() >= 2 and id(p) not in keep32:
                p.data = p.data.to(dtype)
        for layer in model.layers:
            if isinstance(layer.mlp, VitinexDenseMLP):
                layer.mlp.in_proj.bias.data = layer.mlp.in_proj.bias.data.to(dtype)
                layer.mlp.down.bias.data = layer.mlp.down.bias.data.to(dtype)
        model.load_checkpoint_tensors(tensors)
        return model.to(device).eval()
