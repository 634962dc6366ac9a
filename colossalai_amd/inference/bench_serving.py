"""Serving throughput of the ragged-step models next to a Llama of equal width,
depth and per-token work, all through ``ContinuousBatchEngine``: prefill tokens/s
of one long prompt and decode tokens/s of a batch of running sequences. Random
weights, synthetic tokens. Four comparisons: the Kipirax hybrid (paged window
attention + recurrent state), Mubutar (sink-softmax attention with shared
keys, routed experts), Vitinex (latent attention + state-space layers in a
looped block, routed experts) and Tarulix (windowed attention with a distance
table and a learned sink; window + block summaries + talking heads beside a
selective scan; gated experts with identity experts), the last two also next to
Mubutar, whose kernels are the closest.
"""

import json
import time
from typing import Dict, List

import torch

from ..models import (KipiraxConfig, KipiraxForCausalLM, LlamaConfig, LlamaForCausalLM, MubutarConfig,
                      MubutarForCausalLM, TarulixConfig, TarulixForCausalLM, VitinexConfig, VitinexForCausalLM)
from .config import InferenceConfig
from .paged_engine import ContinuousBatchEngine

__all__ = ["SIZES", "hybrid_config", "llama_config", "moe_config", "latent_config", "pooled_config",
           "run_serving_comparison"]

# width, layers, heads, kv_heads, head size, vocab
SIZES = {
    "w2048": dict(width=2048, layers=8, heads=16, kv_heads=4, dim=128, vocab=32000),
    "w4096": dict(width=4096, layers=4, heads=32, kv_heads=8, dim=128, vocab=32000),
}


def hybrid_config(s: dict, max_positions: int, window: int = 1024, keep_first: int = 4) -> KipiraxConfig:
    W, H, G, D = s["width"], s["heads"], s["kv_heads"], s["dim"]
    left = dict(dim=D, heads=H, kv_heads=G, vdim=D, scale=D ** -0.5, mask=dict(size=window, keep_first=keep_first))
    right = dict(dim=D // 2, heads=H // 2, vdim=D)
    delta = dict(conv=4, dim=D, heads=H, kv_heads=H, vdim=D, decay_rank=W // 16, gate_rank=W // 16)
    layers = []
    for i in range(s["layers"]):
        mixer = dict(left=left, right=right) if i % 2 == 0 else delta
        layers.append(dict(type="parallel" if i % 2 == 0 else "channel_delta", mixer=mixer,
                           mlp=dict(kind="dense", ff=4 * W)))
    return KipiraxConfig(vocab=s["vocab"], width=W, max_positions=max_positions, layers=layers, norm_eps=1e-6,
                         norm_groups=4, logit_softcap=30.0)


def _inter(width: int) -> int:
    return (8 * width // 3 + 255) // 256 * 256


def moe_config(s: dict, experts: int = 32, top: int = 6) -> MubutarConfig:
    """Even layers: own keys + dense gated feed-forward of Llama's size. Odd layers: the keys of
    the layer before + routed experts whose active matrices (top experts + shared, two matrices
    each) do the work of Llama's three."""
    W, H, G, D = s["width"], s["heads"], s["kv_heads"], s["dim"]
    inter = _inter(W)
    ff = W // 2
    shared = (3 * inter // 2 - top * ff + 127) // 128 * 128
    att = dict(dim=D, heads=H, kv_heads=G, vdim=D, scale=D ** -0.5, softcap=30.0)
    layers = []
    for i in range(s["layers"]):
        if i % 2 == 0:
            layers.append(dict(type="attention", mixer=att, mlp=dict(kind="dense", ff=inter)))
        else:
            layers.append(dict(type="attention", mixer=dict(att, kv_from=i - 1),
                               mlp=dict(kind="moe", expert=dict(ff=ff), shared=dict(ff=shared),
                                        router=dict(experts=experts, top=top, groups=dict(count=8, keep=4)))))
    return MubutarConfig(vocab=s["vocab"], width=W, layers=layers, norm_eps=1e-6, embedding_scale=W ** 0.5,
                         logit_scale=1.0)


def latent_config(s: dict, experts: int = 32, top: int = 6) -> VitinexConfig:
    """As many layer runs as the size has layers: latent attention and state-space layers in turn, the first two
    looped twice. Per head 64 plain + 64 rotated key channels and 128 value channels (Llama's head size), a latent
    of a quarter of Llama's keys + values per token; the state-space layers are twice the width inside, heads of
    64 channels, a state of 128 per head in 8 groups. Even layers carry Llama's dense feed-forward, odd ones
    Mubutar's expert sizes."""
    W, H, D = s["width"], s["heads"], s["dim"]
    inter = _inter(W)
    ff = W // 2
    shared = (3 * inter // 2 - top * ff + 127) // 128 * 128
    lat = dict(dim=D // 2, rot_dim=D // 2, vdim=D, heads=H, kv_rank=2 * D, q_rank=3 * W // 8,
               rot=dict(base=10000.0, dims=D // 2), scale=D ** -0.5)
    ssm = dict(conv=4, groups=8, heads=2 * W // 64, norm_groups=8, state=128, vdim=64)
    layers = []
    for i in range(s["layers"] - 2):
        mixer = ("latent_attention", lat) if i % 2 == 0 else ("mamba2", ssm)
        mlp = dict(kind="dense", ff=inter) if i % 2 == 0 else dict(
            kind="moe", expert=dict(ff=ff), shared=dict(ff=shared), router=dict(experts=experts, top=top))
        layers.append(dict(type=mixer[0], mixer=mixer[1], mlp=mlp))
    return VitinexConfig(vocab=s["vocab"], width=W, layers=layers, norm_eps=1e-6, residual_mult=0.5,
                         loop=dict(start=0, stop=2, times=2))


def pooled_config(s: dict, experts: int = 32, top: int = 6, window: int = 1024, pool: int = 64) -> TarulixConfig:
    """Windowed attention (distance table of 16 rows, learned sink, values mixed with the first layer's) and the
    parallel mixer (window + summaries of 64 positions + talking heads beside a selective scan of twice the width
    inside, 16 state places, 4 taps) in turn, Llama's head sizes; every layer carries routed gated experts of
    Mubutar's sizes (three matrices each, so two thirds of its hidden width) plus two identity experts."""
    W, H, G, D = s["width"], s["heads"], s["kv_heads"], s["dim"]
    inter = _inter(W)
    ff = W // 3 // 32 * 32
    shared = (inter - top * ff + 127) // 128 * 128
    att = dict(bias_max=float(window), dim=D, heads=H, kv_heads=G, vdim=D, scale=1.0, mask=dict(size=window), v_mix=True)
    left = dict(dim=D, heads=H, kv_heads=G, vdim=D, scale=1.0, softcap=30.0, mask=dict(size=window, pool=pool),
                rot=dict(base=10000.0, dims=D // 2))
    right = dict(conv=4, dt_rank=W // 16, inner=2 * W, state=16)
    mlp = dict(kind="moe", expert=dict(ff=ff), shared=dict(ff=shared), router=dict(experts=experts, identity=2, top=top))
    layers = [dict(type="attention", mixer=att, mlp=mlp) if i % 2 == 0 else
              dict(type="parallel", mixer=dict(left=left, right=right, left_scale=0.7, right_scale=0.6), mlp=mlp)
              for i in range(s["layers"])]
    return TarulixConfig(vocab=s["vocab"], width=W, layers=layers, norm_eps=1e-6)


def llama_config(s: dict, max_positions: int) -> LlamaConfig:
    # gate/up/down of 8/3 W carry the parameters of the hybrid's up/down of 4 W
    inter = _inter(s["width"])
    return LlamaConfig(vocab_size=s["vocab"], hidden_size=s["width"], intermediate_size=inter,
                       num_hidden_layers=s["layers"], num_attention_heads=s["heads"],
                       num_key_value_heads=s["kv_heads"], max_position_embeddings=max_positions)


def _random(model: torch.nn.Module, dtype) -> torch.nn.Module:
    model = model.to(device="cuda")
    with torch.no_grad():
        for p in model.parameters():
            if p.dim() >= 2:
                p.data = p.data.to(dtype)
                p.normal_(0, 0.02)
    return model.eval()


def _timed(fn, repeats: int) -> float:
    fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(repeats):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / repeats


def _hybrid_numbers(s: dict, prompt: int, batch: int, context: int, steps: int) -> Dict[str, float]:
    cfg = hybrid_config(s, max_positions=max(prompt, context + steps + 8) + 8)
    return _ragged_numbers(_random(KipiraxForCausalLM(cfg), torch.bfloat16), cfg.vocab, prompt, batch, context, steps)


def _moe_numbers(s: dict, prompt: int, batch: int, context: int, steps: int) -> Dict[str, float]:
    cfg = moe_config(s)
    model = _random(MubutarForCausalLM(cfg), torch.bfloat16)
    for layer in model.layers:  # the router stays float32
        if hasattr(layer.mlp, "router"):
            layer.mlp.router.data = layer.mlp.router.data.float()
        layer.mix.in_proj.bias.data = layer.mix.in_proj.bias.data.to(torch.bfloat16)
    out = _ragged_numbers(model, cfg.vocab, prompt, batch, context, steps)
    return out


def _latent_numbers(s: dict, prompt: int, batch: int, context: int, steps: int) -> Dict[str, float]:
    cfg = latent_config(s)
    model = _random(VitinexForCausalLM(cfg), torch.bfloat16)
    with torch.no_grad():
        model.loop_in.data = model.loop_in.data.float()     # the loop's mix and the routers stay float32
        model.loop_step.data = model.loop_step.data.float()
        for layer in model.layers:
            if hasattr(layer.mlp, "router"):
                layer.mlp.router.data = layer.mlp.router.data.float()
            if hasattr(layer.mlp, "in_proj"):
                layer.mlp.in_proj.bias.data = layer.mlp.in_proj.bias.data.to(torch.bfloat16)
                layer.mlp.down.bias.data = layer.mlp.down.bias.data.to(torch.bfloat16)
            if layer.kind == "mamba2":
                layer.mix.conv.data = layer.mix.conv.data.float().normal_(0, 0.3)
    return _ragged_numbers(model, cfg.vocab, prompt, batch, context, steps)


def _pooled_numbers(s: dict, prompt: int, batch: int, context: int, steps: int) -> Dict[str, float]:
    cfg = pooled_config(s)
    model = _random(TarulixForCausalLM(cfg), torch.bfloat16)
    with torch.no_grad():
        for layer in model.layers:     # what enters scores, routers and the recurrence stays float32
            layer.mlp.router.data = layer.mlp.router.data.float()
            for att in ([layer.mix] if layer.kind == "attention" else [layer.mix.left]):
                att.in_proj.bias.data = att.in_proj.bias.data.to(torch.bfloat16)
                att.o.bias.data = att.o.bias.data.to(torch.bfloat16)
            if layer.kind == "attention":
                layer.mix.rel.data = layer.mix.rel.data.float()
            else:
                layer.mix.left.talk.data = torch.eye(layer.mix.left.H, device="cuda") + layer.mix.left.talk.data.float()
                layer.mix.right.conv.data = layer.mix.right.conv.data.float().normal_(0, 0.3)
                layer.mix.right.A_log.data = layer.mix.right.A_log.data.float()
    return _ragged_numbers(model, cfg.vocab, prompt, batch, context, steps)


def _ragged_numbers(model, vocab: int, prompt: int, batch: int, context: int, steps: int) -> Dict[str, float]:
    page = 64
    blocks = max(prompt, batch * (context + steps + page)) // page + batch + 2
    eng = ContinuousBatchEngine(model, InferenceConfig(max_batch_size=batch + 1), num_blocks=blocks, block_size=page)
    toks = torch.randint(0, vocab, (prompt,)).tolist()

    def prefill():
        eng.run_ragged([("p", toks, [prompt - 1])])
        eng.close_sequence("p")

    t_prefill = _timed(prefill, 3)
    ctx = torch.randint(0, vocab, (batch, context)).tolist()
    eng.run_ragged([(i, ctx[i], [context - 1]) for i in range(batch)])

    def decode():
        eng.run_ragged([(i, [1], [0]) for i in range(batch)])

    t_decode = _timed(decode, steps)
    params = sum(p.numel() for p in model.parameters())
    del eng, model
    torch.cuda.empty_cache()
    return dict(prefill_tok_s=prompt / t_prefill, decode_tok_s=batch / t_decode, decode_ms=t_decode * 1e3, params=params)


def _llama_numbers(s: dict, prompt: int, batch: int, context: int, steps: int) -> Dict[str, float]:
    from .config import GenerationConfig

    cfg = llama_config(s, max_positions=max(prompt, context + steps + 8) + 8)
    model = _random(LlamaForCausalLM(cfg), torch.bfloat16).to(torch.bfloat16)
    icfg = InferenceConfig(max_batch_size=batch, max_input_len=max(prompt, context), max_output_len=steps + 8)
    eng = ContinuousBatchEngine(model, icfg, block_size=16)
    toks = torch.randint(0, cfg.vocab_size, (1, prompt), device="cuda")
    lens = torch.tensor([prompt], device="cuda", dtype=torch.int32)
    pos = torch.arange(prompt, device="cuda").int()

    @torch.inference_mode()
    def prefill():
        eng.kv.allocate(-1, prompt)
        eng._forward(toks, pos, [-1], None, lens, True)
        eng.kv.free(-1)

    t_prefill = _timed(prefill, 3)
    eng._gen = GenerationConfig(max_new_tokens=steps + 4)
    for row in torch.randint(0, cfg.vocab_size, (batch, context)).tolist():
        eng.add_request(row, steps + 4)
    eng.step()  # prefill of the batch + first decode
    t_decode = _timed(eng.step, steps)
    params = sum(p.numel() for p in model.parameters())
    del eng, model
    torch.cuda.empty_cache()
    return dict(prefill_tok_s=prompt / t_prefill, decode_tok_s=batch / t_decode, decode_ms=t_decode * 1e3, params=params)


def run_serving_comparison(sizes: List[str], prompt: int = 4096, batch: int = 16, context: int = 1024,
                           steps: int = 32, kind: str = "hybrid") -> dict:
    """``kind``: "hybrid" (Kipirax), "moe" (Mubutar), "latent" (Vitinex) or "pooled" (Tarulix), each next to
    Llama; "latent" and "pooled" also next to Mubutar."""
    ours = {"hybrid": _hybrid_numbers, "moe": _moe_numbers, "latent": _latent_numbers, "pooled": _pooled_numbers}[kind]
    out = {}
    for name in sizes:
        s = SIZES[name]
        out[name] = {kind: ours(s, prompt, batch, context, steps)}
        if kind in ("latent", "pooled"):
            out[name]["moe"] = _moe_numbers(s, prompt, batch, context, steps)
        out[name]["llama"] = _llama_numbers(s, prompt, batch, context, steps)
        out[name]["shape"] = dict(s, prompt=prompt, batch=batch, context=context)
    return out
