"""Kumudra, written out plainly in 64-bit: whole sequences, no cache, no batching, one function per mechanism.
It shares nothing with ``ullm_amd``; the GPU tests compare the framework with it.

A model is (config dict as in config.json, {tensor name: 64-bit tensor}).  Linear weights are [out, in].
"""
import math

import torch

F = torch.float64


# ----------------------------------------------------------------------------- small pieces

def layer_norm(x, gain, eps):
    """(x - mean) / sqrt(mean of squared deviations + eps) * gain, over the last axis."""
    mean = x.mean(-1, keepdim=True)
    dev = x - mean
    return dev / torch.sqrt((dev * dev).mean(-1, keepdim=True) + eps) * gain


def unit_rms(x, eps):
    """x over its root mean square (eps inside the root), over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


# ----------------------------------------------------------------------------- rotation

def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims) for i < dims/2; with ``scaling`` (factor, low, high, original) pairs whose wavelength
    2 pi / f is longer than original/low turn ``factor`` times slower, those shorter than original/high are kept,
    and in between the two are blended linearly in original/wavelength."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling is not None:
            factor, low, high, original = scaling
            wavelength = 2 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=F)


def rotate(x, positions, freqs):
    """x [T, heads, dim]: dim i is paired with i + dims/2 over the first dims = 2 len(freqs) dims of each head."""
    half = len(freqs)
    if half == 0:
        return x
    angle = positions.to(F)[:, None] * freqs[None, :]               # [T, half]
    c, s = angle.cos()[:, None, :], angle.sin()[:, None, :]
    a, b = x[..., :half], x[..., half:2 * half]
    return torch.cat((a * c - b * s, b * c + a * s, x[..., 2 * half:]), dim=-1)


# ----------------------------------------------------------------------------- mixers

def windowed_attention(h, w, p, m):
    """Grouped-query softmax attention with biases on q, k, v, a partial rotation and a sliding window."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m.get("vdim", m["dim"])
    q = (h @ w[p + ".q"].T + w[p + ".q.b"]).view(T, H, d)
    k = (h @ w[p + ".k"].T + w[p + ".k.b"]).view(T, G, d)
    v = (h @ w[p + ".v"].T + w[p + ".v.b"]).view(T, G, dv)
    rot = m.get("rot")
    pos = torch.arange(T)
    if rot:
        sc = rot.get("scaling")
        freqs = rotary_frequencies(rot["dims"], rot["base"],
                                   None if not sc else (sc["factor"], sc["low"], sc["high"], sc["original"]))
        q, k = rotate(q, pos, freqs), rotate(k, pos, freqs)
    window = (m.get("mask") or {}).get("size", 0)
    out = torch.zeros(T, H, dv, dtype=F)
    for head in range(H):
        g = head // (H // G)
        scores = (q[:, head] @ k[:, g].T) * m["scale"]              # [query, key]
        dist = pos[:, None] - pos[None, :]
        seen = (dist >= 0) & ((dist < window) if window else torch.ones_like(dist, dtype=torch.bool))
        scores = scores.masked_fill(~seen, -math.inf)
        out[:, head] = torch.softmax(scores, dim=-1) @ v[:, g]
    return out.reshape(T, H * dv) @ w[p + ".o"].T


def decayed_state_outputs(q, k, v, decay, bonus=None):
    """Per head a matrix state S [dim, vdim] from zero.  q, k [T, heads, dim], v [T, heads, vdim], decay [T, heads, dim].
    Without ``bonus``: S_t = diag(decay_t) S_(t-1) + k_t v_t^T and o_t = S_t^T q_t.  With ``bonus`` [heads, dim]:
    o_t = (S_(t-1) + diag(bonus) k_t v_t^T)^T q_t first, then the same update."""
    T, H, d = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, d, dv, dtype=F)
    out = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]                    # [heads, dim, vdim]
        if bonus is None:
            S = decay[t][:, :, None] * S + kv
            out[t] = torch.einsum("hdv,hd->hv", S, q[t])
        else:
            out[t] = torch.einsum("hdv,hd->hv", S + bonus[:, :, None] * kv, q[t])
            S = decay[t][:, :, None] * S + kv
    return out


def time_mixing(h, w, p, m, eps):
    """The recurrent half of a parallel mixer: every projection reads its own blend of the token's and the previous
    token's input; a decay per head and key channel from a small two-layer product; a bonus for the current token."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    prev = torch.cat((torch.zeros(1, h.shape[1], dtype=F), h[:-1]), dim=0)
    mix = {s: h + (prev - h) * w[f"{p}.mu.{s}"] for s in "rkvgw"}
    r = (mix["r"] @ w[p + ".r"].T).view(T, H, d)
    k = (mix["k"] @ w[p + ".k"].T).view(T, H, d)
    v = (mix["v"] @ w[p + ".v"].T).view(T, H, d)
    gate = silu(mix["g"] @ w[p + ".g"].T)
    decay = torch.exp(-torch.exp(torch.tanh(mix["w"] @ w[p + ".w1"].T) @ w[p + ".w2"].T + w[p + ".w0"])).view(T, H, d)
    o = decayed_state_outputs(r, k, v, decay, bonus=w[p + ".u"])
    o = unit_rms(o, eps).reshape(T, H * d) * w[p + ".norm"] * gate
    return o @ w[p + ".o"].T


def parallel_mixer(h, w, p, m, eps):
    left = windowed_attention(h, w, p + ".left", m["left"])
    right = time_mixing(h, w, p + ".right", m["right"], eps)
    return m["left_scale"] * left + m["right_scale"] * right


def gla_mixer(h, w, p, m, eps):
    """Gated linear attention: a decay per key channel sigmoid(z)^(1/tau) from a low-rank product with a bias."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w[p + ".q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w[p + ".k"].T).view(T, H, d)
    v = (h @ w[p + ".v"].T).view(T, H, dv)
    z = (h @ w[p + ".a1"].T) @ w[p + ".a2"].T + w[p + ".a2.b"]
    decay = torch.sigmoid(z).pow(1.0 / m["tau"]).view(T, H, d)
    o = decayed_state_outputs(q, k, v, decay)
    o = unit_rms(o, eps) * w[p + ".norm"]                           # per head, the gain shared by the heads
    return (o.reshape(T, H * dv) * silu(h @ w[p + ".g"].T)) @ w[p + ".o"].T


def lightning_mixer(h, w, p, m, eps):
    """Linear attention with one constant decay per head; silu on q, k and v, a sigmoid gate behind the norm."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[p + ".q"].T).view(T, H, d)
    k = silu(h @ w[p + ".k"].T).view(T, H, d)
    v = silu(h @ w[p + ".v"].T).view(T, H, dv)
    decay = torch.tensor(m["decay"], dtype=F)[None, :, None].expand(T, H, d)
    o = decayed_state_outputs(q, k, v, decay).reshape(T, H * dv)
    o = unit_rms(o, eps) * w[p + ".norm"]                           # all heads together
    return (o * torch.sigmoid(h @ w[p + ".g"].T)) @ w[p + ".o"].T


MIXERS = {"parallel": parallel_mixer, "gla": gla_mixer, "lightning": lightning_mixer}


# ----------------------------------------------------------------------------- feed-forwards

MARGINS = None      # a list: every routed layer run appends, per token, the gap between the last taken and the first left choice score


def gated_unit(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def dense_ff(h, w, p, f):
    return gated_unit(h, w[p + ".gate"], w[p + ".up"], w[p + ".down"])


def routed_ff(h, w, p, f):
    """Sigmoid scores; the choice by score + correction; weights = chosen scores over their sum, times a scale."""
    n, top, scale = f["router"]["experts"], f["router"]["top"], f["router"].get("scale", 1.0)
    s = torch.sigmoid(h @ w[p + ".router"].T)
    choice = s + w[p + ".correction"]
    order = torch.sort(choice, dim=-1, descending=True, stable=True)
    picked = order.indices[:, :top]
    if MARGINS is not None:
        vals = order.values
        MARGINS.append(vals[:, top - 1] - vals[:, top] if top < n else torch.full((h.shape[0],), math.inf, dtype=F))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen = s[t, picked[t]]
        weights = chosen / (chosen.sum() + 1e-20) * scale
        for e, wt in zip(picked[t].tolist(), weights):
            out[t] += wt * gated_unit(h[t], w[f"{p}.e{e}.gate"], w[f"{p}.e{e}.up"], w[f"{p}.e{e}.down"])
    return out


def feed_forward(h, w, p, f):
    return dense_ff(h, w, p, f) if f["kind"] == "dense" else routed_ff(h, w, p, f)


# ----------------------------------------------------------------------------- the model

def run_order(cfg):
    """Layer indices in the order they run: layers start .. stop-1 of ``loop`` ``times`` times in a row."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop["stop"] <= loop["start"]:
        return list(range(n))
    a, b = loop["start"], loop["stop"]
    return list(range(a)) + list(range(a, b)) * loop["times"] + list(range(b, n))


def hyper_sublayer(xs, fn, w, p, q, mult):
    """xs [streams, T, width]: the sublayer reads sum_s in[s] x_s and every new stream t is sum_s mix[s, t] x_s +
    mult * out[t] * y, all from the old streams."""
    u = torch.einsum("s,std->td", w[f"{p}.hc{q}.in"], xs)
    y = fn(u)
    return torch.einsum("sr,std->rtd", w[f"{p}.hc{q}.mix"], xs) + mult * w[f"{p}.hc{q}.out"][:, None, None] * y[None]


def forward(w, cfg, tokens, layers_out=None, round_to=None):
    """Logits [T, vocab] of one sequence from its first token; ``layers_out`` receives the stream (the sum of the
    streams) after every layer run.  With ``round_to`` every sublayer's input is rounded to that dtype on its way
    (what a model loses at the least when its products read such inputs)."""
    rounded = (lambda t: t.to(round_to).to(F)) if round_to is not None else (lambda t: t)
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    streams = cfg.get("streams", 1)
    x = w["embed"][torch.tensor(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    xs = x[None].repeat(streams, 1, 1) if streams > 1 else None
    for i in run_order(cfg):
        L, p = cfg["layers"][i], f"l{i}"
        mixer = lambda u: MIXERS[L["type"]](rounded(layer_norm(u, w[p + ".norm1"], eps)), w, p + ".mix", L["mixer"], eps)   # noqa: E731
        ff = lambda u: feed_forward(rounded(layer_norm(u, w[p + ".norm2"], eps)), w, p + ".mlp", L["mlp"])                    # noqa: E731
        if streams > 1:
            xs = hyper_sublayer(xs, mixer, w, p, 1, mult)
            if L.get("mlp"):
                xs = hyper_sublayer(xs, ff, w, p, 2, mult)
            x = xs.sum(0)
        else:
            x = x + mult * mixer(x)
            if L.get("mlp"):
                x = x + mult * ff(x)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rounded(layer_norm(x, w["final.norm"], eps)) @ w["embed"].T


# ----------------------------------------------------------------------------- random weights

def tensor_shapes(cfg):
    """{tensor name: shape} of a model of this configuration."""
    W, out = cfg["width"], {"embed": (cfg["vocab"], cfg["width"]), "final.norm": (cfg["width"],)}
    S = cfg.get("streams", 1)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}", L["mixer"]
        out[p + ".norm1"] = (W,)
        if L["type"] == "gla":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            rank = m.get("rank", 16)
            out.update({p + ".mix.q": (H * d, W), p + ".mix.k": (H * d, W), p + ".mix.v": (H * dv, W), p + ".mix.g": (H * dv, W),
                        p + ".mix.o": (W, H * dv), p + ".mix.norm": (dv,), p + ".mix.a1": (rank, W), p + ".mix.a2": (H * d, rank),
                        p + ".mix.a2.b": (H * d,)})
        elif L["type"] == "lightning":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            out.update({p + ".mix.q": (H * d, W), p + ".mix.k": (H * d, W), p + ".mix.v": (H * dv, W), p + ".mix.g": (H * dv, W),
                        p + ".mix.o": (W, H * dv), p + ".mix.norm": (H * dv,)})
        else:
            a, r = m["left"], m["right"]
            H, G, d, dv = a["heads"], a["kv_heads"], a["dim"], a.get("vdim", a["dim"])
            q = p + ".mix.left"
            out.update({q + ".q": (H * d, W), q + ".q.b": (H * d,), q + ".k": (G * d, W), q + ".k.b": (G * d,),
                        q + ".v": (G * dv, W), q + ".v.b": (G * dv,), q + ".o": (W, H * dv)})
            q, H, d = p + ".mix.right", r["heads"], r["dim"]
            rank = r.get("rank", 16)
            out.update({f"{q}.mu.{s}": (W,) for s in "rkvgw"})
            out.update({q + ".r": (H * d, W), q + ".k": (H * d, W), q + ".v": (H * d, W), q + ".g": (H * d, W),
                        q + ".w1": (rank, W), q + ".w2": (H * d, rank), q + ".w0": (H * d,), q + ".u": (H, d),
                        q + ".norm": (H * d,), q + ".o": (W, H * d)})
        f = L.get("mlp")
        if f:
            out[p + ".norm2"] = (W,)
            if f["kind"] == "dense":
                out.update({p + ".mlp.gate": (f["ff"], W), p + ".mlp.up": (f["ff"], W), p + ".mlp.down": (W, f["ff"])})
            else:
                n, ff = f["router"]["experts"], f["expert"]["ff"]
                out.update({p + ".mlp.router": (n, W), p + ".mlp.correction": (n,)})
                for e in range(n):
                    out.update({f"{p}.mlp.e{e}.gate": (ff, W), f"{p}.mlp.e{e}.up": (ff, W), f"{p}.mlp.e{e}.down": (W, ff)})
        if S > 1:
            for q in (1, 2) if f else (1,):
                out.update({f"{p}.hc{q}.in": (S,), f"{p}.hc{q}.out": (S,), f"{p}.hc{q}.mix": (S, S)})
    return out


def random_weights(cfg, seed, std=None):
    """bfloat16 tensors of a model of this configuration, sized so that every mechanism matters in the logits."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    S = cfg.get("streams", 1)
    for name, shape in tensor_shapes(cfg).items():
        last = name.rsplit(".", 1)[-1]
        r = torch.randn(shape, generator=g)
        if last in ("norm1", "norm2", "norm") and name != "final.norm" or name == "final.norm":
            t = 1.0 + 0.2 * r
        elif ".hc" in name:
            if last == "mix":
                t = torch.eye(S) * 0.8 + 0.2 / S + 0.1 * r
            elif last == "in":
                t = 1.0 / S + 0.2 * r
            else:
                t = 1.0 + 0.2 * r
        elif ".mu." in name:
            t = torch.rand(shape, generator=g)
        elif last == "w0":
            t = -1.5 + 1.0 * r                                       # decays exp(-exp(w0 + ...)) spread over (0, 1)
        elif last == "u":
            t = 0.5 * r
        elif name.endswith("a2.b"):
            t = 2.0 + 2.0 * r
        elif last == "correction":
            t = 0.1 * r
        elif last == "b":
            t = 0.3 * r
        elif name == "embed":
            t = r
        elif last in ("w2", "a2"):
            t = r * (std if std is not None else 0.5)
        else:
            t = r * (std if std is not None else 1.2 / math.sqrt(shape[-1]))
        out[name] = t.to(torch.bfloat16)
    return out


def greedy_generate(w, cfg, prompt, n):
    """The n tokens that follow ``prompt`` when the largest logit is taken every time (the lowest index on a tie)."""
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(torch.argmax(forward(w, cfg, toks)[-1]))
        toks.append(nxt)
        out.append(nxt)
    return out
