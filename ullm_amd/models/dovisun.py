"""Dovisun as a plan.  Every layer is a parallel block: one RMS norm whose output both the mixer and the feed-forward
read.  Mixers: grouped-query attention without positions, with queries and keys of unit root mean square per head
and a softmax whose denominator holds one more term exp(0); or latent attention with a rotated part whose
frequencies are stretched by wavelength and a sigmoid gate per head.  Feed-forwards: down(relu(up)^2), or experts
picked by the largest router logits (+ a bias) and weighed by the softmax over the picked.  Layers ``loop.start ..
loop.stop - 1`` are passed ``loop.times`` times on the same tensors, every pass with caches of its own, and ahead of
every pass the stream is mixed with the embedding output by ``loop.in``.  The logits are soft-capped.
Tensor names: ``embed``, ``loop.in``, ``l<i>.norm1``, ``l<i>.mix.q / k / v / o`` or ``l<i>.mix.dq / dq.norm / uq / dkv /
dkv.norm / uk / uv / g / o``, ``l<i>.mlp.up / down`` or ``l<i>.mlp.router / router.b / e<j>.gate|up|down``,
``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config.model_config import DovisunAttention, DovisunConfig, DovisunDense, DovisunExperts
from .model import Choice, ModelPlan
from .registry import register_architecture

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o"}
SINK_SCORE = 0.0             # the one more term of the softmax's denominator is exp(0)


def dovisun_plan(cfg: DovisunConfig) -> ModelPlan:
    H, eps = cfg.hidden_size, cfg.norm_eps
    layers = []
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}", L.mixer
        if isinstance(m, DovisunAttention):
            mixer = Choice("mixer", "gqa_attention", dict(
                hidden_size=H, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim,
                prefix=f"{p}.mix", position=None, scale=m.scale, qk_norm="head", qk_norm_eps=eps, qk_norm_gain=False,
                sink_value=SINK_SCORE, names=ATTENTION_NAMES))
        else:
            position = None
            if m.rot_dim:
                sc = m.rot_scaling
                position = Choice("position", "rotary", dict(
                    head_dim=m.rot_dim, theta=m.rot_base, rotary_dim=m.rot_dim, pairing="half", max_positions=None,
                    scaling=None if sc is None else (sc.factor, sc.original, sc.fast, sc.slow)))
            mixer = Choice("mixer", "latent_attention", dict(
                hidden_size=H, num_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim, value_dim=m.vdim, q_rank=m.q_rank,
                kv_rank=m.kv_rank, scale=m.scale, norm_eps=eps, prefix=f"{p}.mix", position=position, head_gate=True))
        params = dict(norm=Choice("norm", "rmsnorm", dict(size=H, eps=eps, weight_name=f"{p}.norm1")), mixer=mixer)
        f = L.mlp
        if isinstance(f, DovisunDense):
            params["ffn"] = Choice("ffn", "mlp", dict(hidden_size=H, intermediate_size=f.ff, prefix=f"{p}.mlp",
                                                      activation="relu2", names={"up": "up", "down": "down"}))
        elif isinstance(f, DovisunExperts):
            params["ffn"] = Choice("ffn", "routed_experts", dict(
                hidden_size=H, experts=f.experts, intermediate_size=f.ff, top=f.top, limit=None, prefix=f"{p}.mlp",
                routing="top_logits", correction=True, names={"correction": "router.b"}))
        layers.append(Choice("block", "parallel", params))
    n = len(layers)
    if cfg.has_loop or cfg.loops:
        # one more "layer": the step ahead of every pass (declared with the tensor also where no layer is passed)
        layers.append(Choice("block", "mix_in_embedding", dict(hidden_size=H, weight_name="loop.in")))
    if cfg.loops:
        # its entries in the run order keep nothing; the passes' layers get cache ids of their own (the first pass
        # the layers' own numbers, later passes numbers behind them)
        order, next_id = [(i, i) for i in range(cfg.loop_start)], n + 1
        for turn in range(cfg.loop_times):
            order.append((n, next_id))
            next_id += 1
            for i in range(cfg.loop_start, cfg.loop_stop):
                order.append((i, i) if turn == 0 else (i, next_id))
                next_id += turn > 0
        order += [(i, i) for i in range(cfg.loop_stop, n)]
    elif cfg.has_loop:
        order = [(i, i) for i in range(n)]       # the declared step is never run
    else:
        order = None
    return ModelPlan(
        vocab_size=cfg.vocab_size, hidden_size=H, embedding_weight="embed", layers=layers,
        final_norm=Choice("norm", "rmsnorm", dict(size=H, eps=eps, weight_name="final.norm")),
        head_weight="head", embedding_scale=cfg.embedding_scale, logit_softcap=cfg.logit_softcap, run_order=order,
        init_std=0.05)


register_architecture("Dovisun", DovisunConfig.from_dict, dovisun_plan)
