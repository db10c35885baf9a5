"""Kumudra as a plan.  The residual stream is kept in ``streams`` copies; every layer is a pre-norm block over them
(layer norms without a bias): a mixer, then a dense or routed feed-forward or none, each reading one mix of the copies
and writing back into all of them, times ``residual_mult``.  Mixers: gated linear attention (a decay per key channel
from a low-rank product), lightning attention (one constant decay per head), or two mixers side by side on the same
input, windowed grouped-query attention with biases and a partly rotated head whose frequencies are stretched by
wavelength beside token-shifted time mixing with a bonus for the current token, added with two weights.  Routed
feed-forwards score their experts by sigmoids, choose by score + correction and scale the normalised weights.  Layers
``loop.start .. loop.stop - 1`` are passed ``loop.times`` times on the same tensors, every pass with caches and state of
its own.  The head is the embedding table (without the embedding's scale).
Tensor names: ``embed``, ``l<i>.norm1 / norm2``, ``l<i>.hc1|hc2.in / out / mix``, ``l<i>.mix.q / k / v / g / o / norm / a1 / a2 /
a2.b`` (gla), ``l<i>.mix.q / k / v / g / o / norm`` (lightning), ``l<i>.mix.left.q / q.b / k / k.b / v / v.b / o`` and
``l<i>.mix.right.mu.r|k|v|g|w / r / k / v / g / w1 / w2 / w0 / u / norm / o`` (parallel), ``l<i>.mlp.gate / up / down`` or
``l<i>.mlp.router / correction / e<j>.gate|up|down``, ``final.norm``.
"""
from __future__ import annotations

from ..config.model_config import KumudraConfig, KumudraDense, KumudraExperts, KumudraGLA, KumudraLightning, KumudraParallel
from .model import Choice, ModelPlan
from .registry import register_architecture

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b"}
SWIGLU_NAMES = {"gate": "gate", "up": "up", "down": "down", "gate_up": "gate_up"}


def _mixer(m, prefix: str, H: int, eps: float) -> Choice:
    if isinstance(m, KumudraGLA):
        return Choice("mixer", "gated_linear_attention", dict(
            hidden_size=H, heads=m.heads, key_dim=m.dim, value_dim=m.vdim, tau=m.tau, norm_eps=eps, prefix=prefix, rank=m.rank))
    if isinstance(m, KumudraLightning):
        return Choice("mixer", "lightning_attention", dict(
            hidden_size=H, heads=m.heads, key_dim=m.dim, value_dim=m.vdim, decay=m.decay, norm_eps=eps, prefix=prefix))
    assert isinstance(m, KumudraParallel)
    a, r = m.left, m.right
    position = None
    if a.rot_dims:
        sc = a.rot_scaling
        position = Choice("position", "rotary", dict(
            head_dim=a.dim, theta=a.rot_base, rotary_dim=a.rot_dims, pairing="half", max_positions=None,
            scaling=None if sc is None else ("by_wavelength", sc.factor, sc.low, sc.high, sc.original)))
    left = Choice("mixer", "gqa_attention", dict(
        hidden_size=H, num_heads=a.heads, num_kv_heads=a.kv_heads, head_dim=a.dim, value_dim=a.vdim, prefix=f"{prefix}.left",
        position=position, bias=True, window=a.window, scale=a.scale, names=ATTENTION_NAMES))
    right = Choice("mixer", "time_mix", dict(hidden_size=H, heads=r.heads, head_dim=r.dim, norm_eps=eps,
                                             prefix=f"{prefix}.right", rank=r.rank))
    return Choice("mixer", "side_by_side", dict(left=left, right=right, left_scale=m.left_scale, right_scale=m.right_scale))


def kumudra_plan(cfg: KumudraConfig) -> ModelPlan:
    H, eps = cfg.hidden_size, cfg.norm_eps
    norm = lambda name: Choice("norm", "layernorm", dict(size=H, eps=eps, weight_name=name))      # noqa: E731
    layers, unused = [], []
    for i, L in enumerate(cfg.layers):
        p = f"l{i}"
        if L.mlp is None:
            # a layer without a feed-forward needs none of that sublayer's tensors; a file may hold them all the same
            unused += [f"{p}.norm2", f"{p}.hc2.in", f"{p}.hc2.out", f"{p}.hc2.mix"]
        params = dict(hidden_size=H, streams=cfg.streams, mixer_norm=norm(f"{p}.norm1"), mixer=_mixer(L.mixer, f"{p}.mix", H, eps),
                      prefix=p, mult=cfg.residual_mult)
        f = L.mlp
        if isinstance(f, KumudraDense):
            params.update(ffn_norm=norm(f"{p}.norm2"),
                          ffn=Choice("ffn", "swiglu", dict(hidden_size=H, intermediate_size=f.ff, prefix=f"{p}.mlp", names=SWIGLU_NAMES)))
        elif isinstance(f, KumudraExperts):
            params.update(ffn_norm=norm(f"{p}.norm2"), ffn=Choice("ffn", "routed_experts", dict(
                hidden_size=H, experts=f.experts, intermediate_size=f.ff, top=f.top, limit=None, prefix=f"{p}.mlp",
                routing="sigmoid", correction=True, weight_scale=f.scale)))
        layers.append(Choice("block", "hyper_prenorm", params))
    # a pass is its layers again with cache ids of their own: the first pass the layers' own numbers, later passes
    # numbers behind them
    order, next_id, n = [], len(layers), len(layers)
    seen = set()
    for i in cfg.run_order():
        if i in seen:
            order.append((i, next_id))
            next_id += 1
        else:
            order.append((i, i))
            seen.add(i)
    return ModelPlan(
        vocab_size=cfg.vocab_size, hidden_size=H, embedding_weight="embed", layers=layers,
        final_norm=norm("final.norm"), head_weight="head", tie_head_to_embedding=True,
        embedding_scale=cfg.embedding_scale, streams=cfg.streams, run_order=order if len(order) != n else None,
        unused_tensors=tuple(unused),
        init_std=0.05)


register_architecture("Kumudra", KumudraConfig.from_dict, kumudra_plan)
