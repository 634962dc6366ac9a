"""Tarulix: a decoder-only language model whose layers norm a sublayer's *output*,
with windowed attention that carries a learned distance table, a learned sink
and value mixing across layers, a mixer that runs attention over a window plus
block summaries beside a selective scan, and softmax-routed gated experts with
identity experts.

Every layer is ``x <- x + g1 * unit(mixer(x))``, then ``x <- x + g2 * unit(ff(x))``:
the sublayers read the float32 residual ``x`` itself, ``unit(y) = y / sqrt(mean(y^2) + eps)``
and the norm's weight ``g`` is one number. The logits are ``head(g * unit(x))``.

* Mixer ``attention``: grouped-query attention with biased projections, no
  rotation; queries and keys divided by their root mean square per head;
  ``score = q.k * scale + table[bucket(i - j), head]`` with logarithmic distance
  buckets; a sliding window; a softmax whose denominator holds one more learned
  term per head (a sink without key or value). In the layers that say ``v_mix``,
  all but the first of them cache ``(1 - l) v + l v_first``, ``v_first`` being
  the first such layer's values of the same token.
* Mixer ``parallel``: ``left_scale * left(x) + right_scale * right(x)``.
  Left: attention with rotary positions on the first ``rot.dims`` channels
  (rotate-half layout), then the per-head unit RMS; a tanh soft cap on the scaled
  score; a window plus one mean key/value per block of ``mask.pool`` positions
  that lies wholly before the window, in one softmax; the heads' softmax weights
  are mixed by a square matrix before each head meets its own values. Right: a
  selective scan (input projection ``[x | z]``, short causal convolution + SiLU,
  projection to ``[dt | B | C]``, a softplus step per channel, the diagonal
  recurrence, ``* silu(z)``, output projection).
* Feed-forward ``moe``: float32 softmax router over real and identity experts,
  choice by score plus a correction, mixing weights = the chosen plain scores
  (not renormalised); experts ``down(silu(gate h) * up h)``; an identity expert
  returns its input; a shared expert of the same form runs for every token.

The module holds the packed layout the kernels want: q/k/v (with biases) of an
attention are one matrix, gate/up of an expert are stacked, the experts are
stacked ``[E, out, in]``. Serving goes through ``forward_ragged`` (a ragged step
over paged keys, block-summary pools and per-sequence state slots); ``forward``
runs whole sequences through the same path with throw-away caches.
"""

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..ops.activation import silu_mul
from ..ops.group_norm import add_scaled_unit_norm, grouped_rms_norm
from ..ops.half_rotary import rotate_halves_unit_norm
from ..ops.paged_attention import (distance_bias_table, mix_values, paged_attention, paged_kv_write, paged_pool_write)
from ..ops.pair_rotary import pair_frequencies
from ..ops.ragged import RaggedBatch
from ..ops.routed_experts import grouped_topk_route, routed_expert_ffn
from ..ops.selective_scan import selective_scan
from ..ops.short_conv import short_conv
from .packed import PackedLinear
from .registry import register_model

__all__ = ["TarulixConfig", "TarulixForCausalLM"]


@dataclass
class TarulixConfig:
    vocab: int
    width: int
    layers: List[dict]
    norm_eps: float = 1e-6

    @classmethod
    def from_dict(cls, d: dict) -> "TarulixConfig":
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=list(d["layers"]),
                   norm_eps=float(d["norm"]["eps"]))

    def to_dict(self) -> dict:
        return {"architecture": "Tarulix", "layers": self.layers, "norm": {"eps": self.norm_eps}, "vocab": self.vocab,
                "width": self.width}


def _scalar(value=1.0):
    return nn.Parameter(torch.tensor(float(value), dtype=torch.float32))


def _vec(n, value=0.0):
    return nn.Parameter(torch.full((n,), value, dtype=torch.float32))


class _Attention(nn.Module):
    """What both attention mixers share: packed biased q/k/v, biased output projection, head sizes, scale, window."""

    def __init__(self, width: int, c: dict, eps: float):
        super().__init__()
        self.H, self.G, self.D, self.Dv = int(c["heads"]), int(c["kv_heads"]), int(c["dim"]), int(c["vdim"])
        if self.H % self.G:
            raise ValueError(f"{self.H} query heads do not split over {self.G} key/value heads")
        self.scale, self.eps = float(c["scale"]), eps
        self.window = int(c["mask"]["size"])
        self.in_proj = PackedLinear(width, {"q": self.H * self.D, "k": self.G * self.D, "v": self.G * self.Dv}, bias=True)
        self.o = nn.Linear(self.H * self.Dv, width, bias=True)

    def kv_shape(self):
        return (self.G, self.D, self.Dv)

    def state_buffers(self):
        return None


class TarulixAttention(_Attention):
    """Windowed attention with a bucketed distance table, a learned sink and cross-layer value mixing."""

    def __init__(self, width: int, c: dict, eps: float, rel_rows: int):
        super().__init__(width, c, eps)
        self.far = float(c["bias_max"])
        self.v_mix = bool(c.get("v_mix", False))
        self.rel = nn.Parameter(torch.zeros(rel_rows, self.H, dtype=torch.float32))
        self.sink = _vec(self.H)
        self.vmix = _scalar(0.0) if self.v_mix else None
        self.summary_block = None
        self._table = None

    def dist_table(self):
        """Bias per distance inside the window, built once from the bucketed rows."""
        if self._table is None or self._table.device != self.rel.device:
            self._table = distance_bias_table(self.rel.detach(), self.far, self.window)
        return self._table

    def forward(self, h, batch: RaggedBatch, pools, state, shared: dict):
        N = h.shape[0]
        p, _ = self.in_proj(h)
        q = rotate_halves_unit_norm(p["q"].view(N, self.H, self.D), batch.positions, None, self.eps)
        k = rotate_halves_unit_norm(p["k"].view(N, self.G, self.D), batch.positions, None, self.eps)
        v = p["v"]
        if self.v_mix:
            if "v_first" in shared:
                v = mix_values(v, shared["v_first"], float(self._lam))
            else:
                shared["v_first"] = v
        kpool, vpool = pools[0], pools[1]
        paged_kv_write(k, v.view(N, self.G, self.Dv), kpool, vpool, batch)
        o = paged_attention(q, kpool, vpool, batch, self.scale, window=self.window, sink_logits=self.sink,
                            dist_bias=self.dist_table())
        return self.o(o.reshape(N, self.H * self.Dv))

    @property
    def _lam(self):
        if not hasattr(self, "_lam_host"):
            self._lam_host = float(self.vmix.detach().float().cpu())
        return self._lam_host


class TarulixPooledAttention(_Attention):
    """Left half of the ``parallel`` mixer: partial rotary, soft cap, window + block summaries, talking heads."""

    def __init__(self, width: int, c: dict, eps: float):
        super().__init__(width, c, eps)
        self.softcap = float(c.get("softcap") or 0.0)
        pool = c["mask"].get("pool")
        self.summary_block = int(pool) if pool else None   # without a block length the window stands alone
        rot = c.get("rot") or {}
        self.rot_dims, self.rot_base = int(rot.get("dims", 0)), float(rot.get("base", 10000.0))
        if self.rot_dims % 2 or self.rot_dims > self.D:
            raise ValueError(f"cannot rotate {self.rot_dims} of {self.D} channels in halves")
        self.register_buffer("freqs", pair_frequencies(self.rot_base, self.rot_dims) if self.rot_dims else None,
                             persistent=False)
        self.talk = nn.Parameter(torch.eye(self.H, dtype=torch.float32))

    def forward(self, h, batch: RaggedBatch, pools, state, shared: dict):
        N = h.shape[0]
        p, _ = self.in_proj(h)
        q = rotate_halves_unit_norm(p["q"].view(N, self.H, self.D), batch.positions, self.freqs, self.eps)
        k = rotate_halves_unit_norm(p["k"].view(N, self.G, self.D), batch.positions, self.freqs, self.eps)
        kpool, vpool, ksum, vsum = pools
        paged_kv_write(k, p["v"].view(N, self.G, self.Dv), kpool, vpool, batch)
        pooled = None
        if self.summary_block is not None:
            paged_pool_write(kpool, vpool, ksum, vsum, batch, self.summary_block)
            pooled = (ksum, vsum, self.summary_block)
        o = paged_attention(q, kpool, vpool, batch, self.scale, window=self.window, softcap=self.softcap,
                            pooled=pooled, talk=self.talk)
        return self.o(o.reshape(N, self.H * self.Dv))


class TarulixSelectiveScan(nn.Module):
    """Right half of the ``parallel`` mixer."""

    def __init__(self, width: int, c: dict):
        super().__init__()
        self.inner, self.S, self.R, self.K = int(c["inner"]), int(c["state"]), int(c["dt_rank"]), int(c["conv"])
        self.in_proj = nn.Linear(width, 2 * self.inner, bias=False)
        self.conv = nn.Parameter(torch.randn(self.inner, self.K, dtype=torch.float32) * 0.5)
        self.conv_b = _vec(self.inner)
        self.x_proj = nn.Linear(self.inner, self.R + 2 * self.S, bias=False)
        self.dt_proj = nn.Linear(self.R, self.inner, bias=False)
        self.dt_bias, self.D_skip = _vec(self.inner), _vec(self.inner, 1.0)
        self.A_log = nn.Parameter(torch.zeros(self.inner, self.S, dtype=torch.float32))
        self.o = nn.Linear(self.inner, width, bias=False)

    def state_buffers(self):
        buf = {"S": (self.inner, self.S)}
        if self.K > 1:
            buf["tail"] = (self.K - 1, self.inner)
        return buf

    def forward(self, h, batch: RaggedBatch, state):
        inner, R, S = self.inner, self.R, self.S
        xz = self.in_proj(h)
        # the convolution feeds a recurrence: its activated output stays float32 for the scan, the projection that
        # follows reads its rounding
        x = short_conv(xz[:, :inner], self.conv, state.get("tail"), batch, True, torch.float32, self.conv_b)
        proj = self.x_proj(x.to(h.dtype))
        dt_raw = self.dt_proj(proj[:, :R])
        y = selective_scan(x, dt_raw, self.A_log, proj[:, R : R + S], proj[:, R + S :], self.D_skip, self.dt_bias,
                           xz[:, inner:], state["S"], batch, h.dtype)
        return self.o(y)


class TarulixParallel(nn.Module):
    def __init__(self, width: int, c: dict, eps: float):
        super().__init__()
        self.left = TarulixPooledAttention(width, c["left"], eps)
        self.right = TarulixSelectiveScan(width, c["right"])
        self.left_scale, self.right_scale = float(c["left_scale"]), float(c["right_scale"])
        self.summary_block = self.left.summary_block

    def kv_shape(self):
        return self.left.kv_shape()

    def state_buffers(self):
        return self.right.state_buffers()


class TarulixExpert(nn.Module):
    """down(silu(gate h) * up h), no biases; gate and up are one matrix."""

    def __init__(self, width: int, ff: int):
        super().__init__()
        self.in_proj = PackedLinear(width, {"gate": ff, "up": ff})
        self.down = nn.Linear(ff, width, bias=False)

    def forward(self, h):
        _, y = self.in_proj(h)
        return self.down(silu_mul(y))


class TarulixMoE(nn.Module):
    def __init__(self, width: int, c: dict):
        super().__init__()
        r = c["router"]
        self.E, self.I, self.top = int(r["experts"]), int(r.get("identity", 0)), int(r["top"])
        ff = int(c["expert"]["ff"])
        self.router = nn.Parameter(torch.randn(self.E + self.I, width, dtype=torch.float32) * width ** -0.5)  # float32 always
        self.correction = _vec(self.E + self.I)
        self.w_up = nn.Parameter(torch.randn(self.E, 2 * ff, width) * width ** -0.5)     # [gate; up] per expert
        self.w_down = nn.Parameter(torch.randn(self.E, width, ff) * ff ** -0.5)
        self.shared = TarulixExpert(width, int(c["shared"]["ff"])) if c.get("shared") else None

    def forward(self, h):
        logits = F.linear(h.float(), self.router)
        ids, weights = grouped_topk_route(logits, self.correction, self.top, score="softmax", renorm=False)
        base = self.shared(h) if self.shared is not None else None
        return routed_expert_ffn(h, self.w_up, self.w_down, ids, weights, base, "silu_gated",
                                 identity=self.I > 0, num_ids=self.E + self.I)


MLPS = {"moe": TarulixMoE}


class TarulixLayer(nn.Module):
    def __init__(self, cfg: TarulixConfig, spec: dict, rel_rows: int):
        super().__init__()
        self.kind = spec["type"]
        if self.kind == "attention":
            self.mix = TarulixAttention(cfg.width, spec["mixer"], cfg.norm_eps, rel_rows)
        elif self.kind == "parallel":
            self.mix = TarulixParallel(cfg.width, spec["mixer"], cfg.norm_eps)
        else:
            raise ValueError(f"unknown mixer type {self.kind!r}")
        self.norm1 = _scalar()
        m = spec.get("mlp")
        if m is not None and m.get("kind", "moe") not in MLPS:
            raise ValueError(f"unknown feed-forward kind {m.get('kind')!r}")
        self.mlp = MLPS[m.get("kind", "moe")](cfg.width, m) if m is not None else None
        self.norm2 = _scalar() if m is not None else None


@register_model("Tarulix")
class TarulixForCausalLM(nn.Module):
    config_class = TarulixConfig
    serves_ragged = True  # the serving engines drive forward_ragged

    def __init__(self, cfg: TarulixConfig, rel_rows: Optional[Dict[int, int]] = None):
        """``rel_rows`` maps a layer index to the rows of its distance table (a checkpoint's tensor shape gives it;
        16 otherwise)."""
        super().__init__()
        self.config = cfg
        self.embed = nn.Embedding(cfg.vocab, cfg.width)
        self.layers = nn.ModuleList([TarulixLayer(cfg, s, (rel_rows or {}).get(i, 16)) for i, s in enumerate(cfg.layers)])
        self.final_norm = _scalar()
        self.head = nn.Linear(cfg.width, cfg.vocab, bias=False)
        first = None
        for i, layer in enumerate(self.layers):
            if layer.kind == "attention" and layer.mix.v_mix:
                if first is None:
                    first = layer.mix
                elif (first.G, first.Dv) != (layer.mix.G, layer.mix.Dv):
                    raise ValueError(f"layer {i} mixes its values with those of a layer of other value sizes")
        self._gains = None

    # ------------------------------------------------------------ cache plan
    def kv_layer_shapes(self):
        """Per layer ``(kv_heads, key_dim, value_dim)``."""
        return [l.mix.kv_shape() for l in self.layers]

    def kv_layer_summaries(self):
        """Per layer the block length whose mean keys and values it also keeps, None for none."""
        return [l.mix.summary_block for l in self.layers]

    def state_layer_buffers(self):
        """Per layer ``{name: shape}`` of float32 state kept per sequence, or None."""
        return [l.mix.state_buffers() for l in self.layers]

    @property
    def act_dtype(self):
        return self.head.weight.dtype

    def _gain_values(self):
        """The norms' single weights as host numbers, fetched once."""
        if self._gains is None:
            vals = [self.final_norm] + [l.norm1 for l in self.layers] + [l.norm2 for l in self.layers if l.norm2 is not None]
            host = torch.stack([v.detach().float() for v in vals]).cpu().tolist()
            n = len(self.layers)
            it = iter(host[1 + n:])
            self._gains = (host[0], host[1 : 1 + n], [next(it) if l.norm2 is not None else None for l in self.layers])
        return self._gains

    # ---------------------------------------------------------------- serve
    def forward_ragged(self, tokens: torch.Tensor, batch: RaggedBatch, kv, state,
                       want: Optional[torch.Tensor] = None, residuals: Optional[list] = None) -> torch.Tensor:
        """tokens [N] (flat, sequence after sequence as ``batch`` says); ``kv`` a KVCacheManager and ``state`` a
        StateCacheManager laid out by ``kv_layer_shapes`` / ``kv_layer_summaries`` / ``state_layer_buffers``.
        Returns float32 logits of the rows ``want`` (indices into the flat token axis; all rows if None).
        ``residuals``, when a list, receives a copy of the float32 residual stream after every layer."""
        cfg, act = self.config, self.act_dtype
        eps = cfg.norm_eps
        g_final, g1, g2 = self._gain_values()
        x = self.embed(tokens).float()
        h = x.to(act)
        shared: dict = {}  # what one layer leaves for later ones within the step (the first mixed values)
        for i, layer in enumerate(self.layers):
            pools = (kv.k_pools[i], kv.v_pools[i], kv.k_summaries[i], kv.v_summaries[i])
            if layer.kind == "parallel":
                a = layer.mix.left(h, batch, pools, None, shared)
                b = layer.mix.right(h, batch, state.layers[i])
                h = add_scaled_unit_norm(x, a, b, layer.mix.left_scale, layer.mix.right_scale, g1[i], eps, act)
            else:
                a = layer.mix(h, batch, pools, None, shared)
                h = add_scaled_unit_norm(x, a, None, 1.0, 0.0, g1[i], eps, act)
            if layer.mlp is not None:
                h = add_scaled_unit_norm(x, layer.mlp(h), None, 1.0, 0.0, g2[i], eps, act)
            if residuals is not None:
                residuals.append(x.clone())
        if want is not None:
            x = x.index_select(0, want)
        ones = x.new_full((cfg.width,), g_final)
        return self.head(grouped_rms_norm(x, ones, 1, eps, None, act)).float()

    def forward(self, input_ids: torch.Tensor) -> torch.Tensor:
        """input_ids [B, S] -> logits [B, S, vocab] (float32), every sequence from position 0 with caches that
        live for this call only."""
        from ..inference.kv_cache import KVCacheManager
        from ..inference.state_cache import StateCacheManager

        B, S = input_ids.shape
        dev = input_ids.device
        page = 16
        pages = (S + page - 1) // page
        kv = KVCacheManager(len(self.layers), 0, 0, num_blocks=B * pages, block_size=page, device=dev,
                            dtype=self.act_dtype, layer_shapes=self.kv_layer_shapes(),
                            layer_summaries=self.kv_layer_summaries())
        state = StateCacheManager(self.state_layer_buffers(), B, device=dev)
        tables = [list(range(b * pages, (b + 1) * pages)) for b in range(B)]
        batch = RaggedBatch.build([S] * B, [0] * B, list(range(B)), dev, tables, page)
        with torch.no_grad():
            return self.forward_ragged(input_ids.reshape(-1), batch, kv, state).view(B, S, -1)

    # -------------------------------------------------------------- weights
    def load_checkpoint_tensors(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Pack a checkpoint's per-projection tensors (``embed``, ``l<i>.norm1|2``, ``l<i>.mix.*``,
        ``l<i>.mlp.*``, ``final.norm``, ``head``) into this module's fused parameters. Every tensor must be used
        and every parameter filled."""
        used = set()

        def get(name):
            used.add(name)
            return tensors[name]

        def put(param, value):
            assert tuple(param.shape) == tuple(value.shape), (tuple(param.shape), tuple(value.shape))
            param.data.copy_(value.to(param.dtype))

        def put_attention(m, p):
            put(m.in_proj.weight, torch.cat([get(p + part) for part in m.in_proj.parts], 0))
            put(m.in_proj.bias, torch.cat([get(p + part + ".b") for part in m.in_proj.parts], 0))
            put(m.o.weight, get(p + "o"))
            put(m.o.bias, get(p + "o.b"))

        put(self.embed.weight, get("embed"))
        put(self.final_norm, get("final.norm"))
        put(self.head.weight, get("head"))
        for i, layer in enumerate(self.layers):
            p, m = f"l{i}.", layer.mix
            put(layer.norm1, get(p + "norm1"))
            if layer.kind == "attention":
                put_attention(m, p + "mix.")
                put(m.rel, get(p + "mix.rel"))
                put(m.sink, get(p + "mix.sink"))
                if m.v_mix:
                    put(m.vmix, get(p + "mix.vmix"))
                elif p + "mix.vmix" in tensors:
                    used.add(p + "mix.vmix")
                m._table = None
                m.__dict__.pop("_lam_host", None)
            else:
                put_attention(m.left, p + "mix.left.")
                put(m.left.talk, get(p + "mix.left.talk"))
                r, q = m.right, p + "mix.right."
                put(r.in_proj.weight, get(q + "in"))
                put(r.conv, get(q + "conv"))
                put(r.conv_b, get(q + "conv.b"))
                put(r.x_proj.weight, get(q + "x"))
                put(r.dt_proj.weight, get(q + "dt"))
                put(r.dt_bias, get(q + "dt.b"))
                put(r.A_log, get(q + "A_log"))
                put(r.D_skip, get(q + "D"))
                put(r.o.weight, get(q + "o"))
            f = layer.mlp
            if f is not None:
                put(layer.norm2, get(p + "norm2"))
                put(f.router, get(p + "mlp.router"))
                put(f.correction, get(p + "mlp.correction"))
                put(f.w_up, torch.stack([torch.cat([get(p + f"mlp.e{e}.gate"), get(p + f"mlp.e{e}.up")], 0)
                                         for e in range(f.E)], 0))
                put(f.w_down, torch.stack([get(p + f"mlp.e{e}.down") for e in range(f.E)], 0))
                if f.shared is not None:
                    put(f.shared.in_proj.weight, torch.cat([get(p + "mlp.shared.gate"), get(p + "mlp.shared.up")], 0))
                    put(f.shared.down.weight, get(p + "mlp.shared.down"))
        self._gains = None
        missing = set(tensors) - used
        if missing:
            raise ValueError(f"checkpoint tensors without a place in the model: {sorted(missing)[:8]}")

    @classmethod
    def from_checkpoint(cls, config: dict, tensors: Dict[str, torch.Tensor], dtype=torch.bfloat16, device="cpu"):
        """Build from a parsed config.json and a name -> tensor mapping. Matrices and projection biases take
        ``dtype``; the norms' weights, the router and its correction, the distance table, sink, head-mixing matrix
        and everything that enters the recurrence (taps, step bias, decay logarithms, direct path) stay float32."""
        rel_rows = {i: int(tensors[f"l{i}.mix.rel"].shape[0]) for i in range(len(config["layers"]))
                    if f"l{i}.mix.rel" in tensors}
        model = cls(TarulixConfig.from_dict(config), rel_rows)
        keep32 = set()
        for l in model.layers:
            if l.mlp is not None:
                keep32.add(id(l.mlp.router))
            if l.kind == "attention":
                keep32.add(id(l.mix.rel))
            else:
                keep32 |= {id(l.mix.left.talk), id(l.mix.right.conv), id(l.mix.right.A_log)}
        for p in model.parameters():
            if p.dim() >= 2 and id(p) not in keep32:
                p.data = p.data.to(dtype)
        for l in model.layers:
            for att in ([l.mix] if l.kind == "attention" else [l.mix.left]):
                att.in_proj.bias.data = att.in_proj.bias.data.to(dtype)
                att.o.bias.data = att.o.bias.data.to(dtype)
        model.load_checkpoint_tensors(tensors)
        return model.to(device).eval()
