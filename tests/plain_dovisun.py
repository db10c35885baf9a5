"""Plain, slow Dovisun: whole sequences, no cache, one function per mechanism, written from the design's
equations.  It shares no code with ``ullm_amd``; the framework is tested against it.

A model is a dict ``cfg`` (the config.json keys) and a dict ``w`` of tensors by checkpoint name.  Everything is
computed in the dtype of ``w`` (the tests widen to float64 for a sharp oracle).

The design: e = embed[token] * s.  Layers ``loop.start .. loop.stop - 1`` run ``loop.times`` times in a row on the
same tensors, the others once; ahead of every pass over the looped layers the stream is mixed with the embedding
again, x <- W_in [x ; e].  Every layer is x <- x + mixer(h) + ff(h) with h = rms(x) * gain, one norm for both
sublayers.  Mixers: grouped-query attention without positions whose queries and keys have unit root mean square per
head and whose softmax has one more term exp(0) in its denominator; and latent attention, whose queries and
keys/values go through small latents, with a rotated part shared by all heads and a sigmoid gate per head on the
output.  Feed-forwards: down(relu(up h)^2), or a router that picks ``top`` of several silu-gated units by its
logits and weighs them by the softmax over the picked logits.  logits = cap * tanh(head rms(x) / cap).
"""
import math
from typing import List, Optional

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def causal(T: int) -> torch.Tensor:
    return torch.arange(T)[:, None] >= torch.arange(T)[None, :]


def softmax_one_more(scores: torch.Tensor) -> torch.Tensor:
    """Rows of ``scores`` (-inf where masked) to weights e^s / (1 + sum e^s)."""
    top = torch.clamp(scores.max(-1, keepdim=True).values, min=0.0)
    e = torch.exp(scores - top)
    return e / (e.sum(-1, keepdim=True) + torch.exp(-top))


def attention(w, prefix: str, m: dict, eps: float, h: torch.Tensor, sink: bool = True) -> torch.Tensor:
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms((h @ w[f"{prefix}.q"].T).view(T, H, d), eps)
    k = rms((h @ w[f"{prefix}.k"].T).view(T, G, d), eps)
    v = (h @ w[f"{prefix}.v"].T).view(T, G, dv)
    heads = []
    for a in range(H):
        g = a // (H // G)
        s = ((q[:, a] @ k[:, g].T) * m["scale"]).masked_fill(~causal(T), -math.inf)
        p = softmax_one_more(s) if sink else torch.softmax(s, -1)
        heads.append(p @ v[:, g])
    return torch.cat(heads, -1) @ w[f"{prefix}.o"].T


def yarn_frequencies(rot: dict) -> (torch.Tensor, float):
    """(frequency of every pair float64 [dims/2], the factor on cos and sin)."""
    dims, base = rot["dims"], float(rot["base"])
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(base, dtype=torch.float64), -2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [T, ..., d]: dim i < dims/2 is paired with dim i + dims/2 and the pair turned by p * f_i; dims from
    ``dims`` on pass unchanged."""
    dims = rot["dims"]
    f, mag = yarn_frequencies(rot)
    angle = positions.to(torch.float64)[:, None] * f
    shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (dims // 2,)
    cos, sin = (angle.cos() * mag).to(x.dtype).view(shape), (angle.sin() * mag).to(x.dtype).view(shape)
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    out = x.clone()
    out[..., :dims // 2] = u * cos - v * sin
    out[..., dims // 2:dims] = v * cos + u * sin
    return out


def latent_attention(w, prefix: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    T = h.shape[0]
    H, d, r, dv, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = rms(h @ w[f"{prefix}.dq"].T, eps) * w[f"{prefix}.dq.norm"]
    q = (cq @ w[f"{prefix}.uq"].T).view(T, H, d + r)
    q_plain, q_rot = q[..., :d], rotate_halves(q[..., d:], pos, m["rot"]) if r else q[..., d:]
    down = h @ w[f"{prefix}.dkv"].T
    c = rms(down[:, :kr], eps) * w[f"{prefix}.dkv.norm"]
    k_rot = rotate_halves(down[:, kr:], pos, m["rot"]) if r else down[:, kr:]   # one for all heads
    k_plain = (c @ w[f"{prefix}.uk"].T).view(T, H, d)
    v = (c @ w[f"{prefix}.uv"].T).view(T, H, dv)
    gate = torch.sigmoid(h @ w[f"{prefix}.g"].T)                           # [T, H]
    heads = []
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * m["scale"]
        p = torch.softmax(s.masked_fill(~causal(T), -math.inf), -1)
        heads.append((p @ v[:, a]) * gate[:, a:a + 1])
    return torch.cat(heads, -1) @ w[f"{prefix}.o"].T


def dense(w, prefix: str, h: torch.Tensor) -> torch.Tensor:
    return torch.relu(h @ w[f"{prefix}.up"].T) ** 2 @ w[f"{prefix}.down"].T


def expert(w, prefix: str, h: torch.Tensor) -> torch.Tensor:
    g = h @ w[f"{prefix}.gate"].T
    return (g * torch.sigmoid(g) * (h @ w[f"{prefix}.up"].T)) @ w[f"{prefix}.down"].T


MARGINS = None      # a list: every routed layer run appends, per row, the gap between the last chosen logit and the next


def route(w, prefix: str, f: dict, h: torch.Tensor):
    """(chosen experts long [T, top], their weights [T, top], logits [T, experts])."""
    z = h @ w[f"{prefix}.router"].T + w[f"{prefix}.router.b"]
    top = torch.topk(z, f["router"]["top"], dim=-1)
    if MARGINS is not None:
        ranked = torch.sort(z, dim=-1, descending=True).values
        k = f["router"]["top"]
        MARGINS.append((ranked[:, k - 1] - ranked[:, k]) if k < z.shape[-1] else torch.full((z.shape[0],), math.inf))
    return top.indices, torch.softmax(top.values, -1), z


def experts(w, prefix: str, f: dict, h: torch.Tensor) -> torch.Tensor:
    ids, weights, _ = route(w, prefix, f, h)
    out = torch.zeros_like(h)
    for e in range(f["router"]["experts"]):
        hit = ids == e
        rows = hit.any(-1)
        if rows.any():
            out[rows] += expert(w, f"{prefix}.e{e}", h[rows]) * (weights * hit)[rows].sum(-1, keepdim=True)
    return out


def layer(w, cfg: dict, i: int, x: torch.Tensor, round_to=None) -> torch.Tensor:
    L, eps, p = cfg["layers"][i], cfg["norm"]["eps"], f"l{i}"
    h = rms(x, eps) * w[f"{p}.norm1"]
    if round_to is not None:
        h = h.to(round_to).to(x.dtype)          # what an engine loses at the least that computes in this type
    if L["type"] == "attention":
        y = attention(w, f"{p}.mix", L["mixer"], eps, h)
    elif L["type"] == "latent_attention":
        y = latent_attention(w, f"{p}.mix", L["mixer"], eps, h)
    else:
        raise ValueError(L["type"])
    f = L.get("mlp")
    if f is not None:
        y = y + (dense(w, f"{p}.mlp", h) if f["kind"] == "dense" else experts(w, f"{p}.mlp", f, h))
    return x + y


def run_order(cfg: dict) -> List[tuple]:
    """[(layer, first of a pass over the looped layers)] in the order the layers run."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(a)]
    for _ in range(times):
        order += [(i, i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def forward(w, cfg: dict, tokens, streams: Optional[list] = None, round_to=None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence; ``streams`` (a list) receives the stream after every layer run.  With
    ``round_to`` the sublayers' common input is rounded to that type and nothing else is."""
    ids = torch.as_tensor(tokens, dtype=torch.long)
    e = w["embed"][ids] * (cfg.get("embedding") or {}).get("scale", 1.0)
    x = e
    for i, mix_in in run_order(cfg):
        if mix_in:
            x = torch.cat((x, e), -1) @ w["loop.in"].T
        x = layer(w, cfg, i, x, round_to)
        if streams is not None:
            streams.append(x)
    z = (rms(x, cfg["norm"]["eps"]) * w["final.norm"]) @ w["head"].T
    cap = cfg.get("logit_softcap") or 0.0
    return cap * torch.tanh(z / cap) if cap > 0 else z


def greedy_generate(w, cfg, prompt: List[int], n: int) -> List[int]:
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(forward(w, cfg, toks)[-1].argmax())
        toks.append(nxt)
        out.append(nxt)
    return out


def random_weights(cfg: dict, seed: int, std: float = 0.08, router_bias_std: float = 0.3):
    """bfloat16 tensors under the design's names.  The router's logits are about a unit and a half wide whatever
    the width and its biases a third of a unit, so that a bias left out or added to the weights moves the choice;
    the mixing matrix ahead of a pass keeps the stream's size."""
    g = torch.Generator().manual_seed(seed)
    H = cfg["width"]

    def mat(*shape, s=std):
        return (torch.randn(*shape, generator=g) * s).bfloat16()

    def gain(n):
        return (1 + 0.2 * torch.randn(n, generator=g)).bfloat16()

    w = {"embed": mat(cfg["vocab"], H, s=0.5), "head": mat(cfg["vocab"], H, s=0.3), "final.norm": gain(H)}
    if cfg.get("loop"):
        w["loop.in"] = mat(H, 2 * H, s=0.7 / math.sqrt(H))
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}", L["mixer"]
        w[f"{p}.norm1"] = gain(H)
        if L["type"] == "attention":
            w[f"{p}.mix.q"], w[f"{p}.mix.k"] = mat(m["heads"] * m["dim"], H, s=0.25), mat(m["kv_heads"] * m["dim"], H, s=0.25)
            w[f"{p}.mix.v"], w[f"{p}.mix.o"] = mat(m["kv_heads"] * m["vdim"], H, s=0.25), mat(H, m["heads"] * m["vdim"])
        else:
            d, r = m["dim"], m["rot_dim"]
            w[f"{p}.mix.dq"], w[f"{p}.mix.dq.norm"] = mat(m["q_rank"], H, s=0.25), gain(m["q_rank"])
            w[f"{p}.mix.uq"] = mat(m["heads"] * (d + r), m["q_rank"], s=0.25)
            w[f"{p}.mix.dkv"], w[f"{p}.mix.dkv.norm"] = mat(m["kv_rank"] + r, H, s=0.25), gain(m["kv_rank"])
            w[f"{p}.mix.uk"], w[f"{p}.mix.uv"] = mat(m["heads"] * d, m["kv_rank"], s=0.25), mat(m["heads"] * m["vdim"], m["kv_rank"], s=0.2)
            w[f"{p}.mix.g"], w[f"{p}.mix.o"] = mat(m["heads"], H, s=0.3), mat(H, m["heads"] * m["vdim"])
        f = L.get("mlp")
        if f is None:
            continue
        if f["kind"] == "dense":
            w[f"{p}.mlp.up"], w[f"{p}.mlp.down"] = mat(f["ff"], H, s=0.25), mat(H, f["ff"])
            continue
        n = f["router"]["experts"]
        w[f"{p}.mlp.router"], w[f"{p}.mlp.router.b"] = mat(n, H, s=1.5 / math.sqrt(H)), mat(n, s=router_bias_std)
        for e in range(n):
            ff = f["expert"]["ff"]
            w[f"{p}.mlp.e{e}.gate"], w[f"{p}.mlp.e{e}.up"] = mat(ff, H, s=0.3), mat(ff, H, s=0.3)
            w[f"{p}.mlp.e{e}.down"] = mat(H, ff)
    return w
