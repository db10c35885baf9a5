"""Kumudra configurations drawn at random (width, copies of the stream, kinds and order of layers, heads, key and value
sizes, windows, rotated dims and their stretching, decays, experts and top counts, layers without a feed-forward, which
layers are passed again and how often) through the replayer: in 32-bit against the plain 64-bit implementation, whole
prompts, portions of drawn sizes followed by single tokens, and a schedule of up to four live requests in a pool and
slots that are used again; in bfloat16 the same schedules against the same logits, most rows to rounding."""
import json
import os
import random

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

import plain_kumudra as plain
from gpu_util import DEV

pytestmark = pytest.mark.gpu


def drawn_mlp(rng):
    kind = rng.random()
    if kind < 0.15:
        return None
    if kind < 0.5:
        return dict(kind="dense", ff=rng.choice([4, 12, 20, 64, 100, 136, 256]))
    experts = rng.choice([1, 2, 3, 5, 8, 16, 40])
    return dict(kind="moe", router=dict(experts=experts, top=rng.randint(1, min(6, experts)), scale=rng.choice([0.5, 1.0, 2.5])),
                expert=dict(ff=rng.choice([4, 6, 8, 12, 16, 24, 40, 64, 100, 130])))


def drawn_layer(rng):
    kind = rng.random()
    if kind < 0.3:
        mixer = dict(heads=rng.choice([1, 2, 3, 4, 8]), dim=rng.choice([4, 6, 8, 16, 32, 40, 64, 128]),
                     vdim=rng.choice([4, 10, 16, 32, 64, 72, 128]), tau=rng.choice([1.0, 4.0, 12.0]), rank=rng.choice([1, 4, 16, 24]))
        return dict(type="gla", mixer=mixer, mlp=drawn_mlp(rng))
    if kind < 0.6:
        heads = rng.choice([1, 2, 3, 4, 8])
        mixer = dict(heads=heads, dim=rng.choice([4, 6, 8, 16, 32, 64, 96, 200]), vdim=rng.choice([4, 10, 16, 32, 64, 128]),
                     decay=[rng.choice([1.0, 0.999, 0.97, 0.8, 0.3]) for _ in range(heads)])
        return dict(type="lightning", mixer=mixer, mlp=drawn_mlp(rng))
    kv = rng.choice([1, 1, 2, 3, 4])
    dim = rng.choice([8, 12, 16, 24, 32, 40, 64, 72, 96, 128, 160, 256])
    left = dict(heads=kv * rng.choice([1, 2, 3, 4, 8]), kv_heads=kv, dim=dim, vdim=rng.choice([dim, dim, 4, 8, 20, 64, 128]),
                scale=rng.choice([0.05, 0.125, 0.3]))
    if rng.random() < 0.8:
        left["mask"] = dict(size=rng.choice([1, 2, 5, 16, 17, 33, 64, 100]))
    if rng.random() < 0.8:
        left["rot"] = dict(base=rng.choice([100.0, 10000.0, 500000.0]), dims=rng.choice([d for d in (2, 4, 8, 16, 32, 64, dim) if d <= dim]))
        if rng.random() < 0.7:
            low = rng.choice([1.0, 2.0])
            left["rot"]["scaling"] = dict(factor=rng.choice([1.0, 2.0, 8.0, 32.0]), low=low, high=low * rng.choice([2.0, 4.0]),
                                          original=rng.choice([16, 64, 512, 4096]))
    right = dict(heads=rng.choice([1, 2, 3, 6]), dim=rng.choice([4, 6, 8, 16, 32, 64]), rank=rng.choice([1, 4, 16, 20]))
    return dict(type="parallel", mlp=drawn_mlp(rng), mixer=dict(left=left, right=right, left_scale=rng.choice([1.0, 0.55, 0.3]),
                                                               right_scale=rng.choice([1.0, 0.8, 1.4])))


def drawn_config(rng):
    layers = [drawn_layer(rng) for _ in range(rng.randint(1, 5))]
    cfg = dict(architecture="Kumudra", vocab=rng.randint(40, 700), layers=layers, norm=dict(eps=rng.choice([1e-5, 1e-6, 1e-3])),
               width=rng.choice([20, 24, 32, 36, 40, 48, 50, 64, 72, 96, 100, 128, 160, 256]), streams=rng.choice([1, 2, 2, 3, 4, 6]))
    if rng.random() < 0.8:
        start = rng.randint(0, len(layers) - 1)
        cfg["loop"] = dict(start=start, stop=rng.randint(start, len(layers)), times=rng.choice([1, 2, 2, 3, 4]))
    if rng.random() < 0.7:
        cfg["embedding"] = dict(scale=rng.choice([0.5, 3.0, 11.0]))
    if rng.random() < 0.7:
        cfg["residual_mult"] = rng.choice([0.3, 0.65, 1.5])
    return cfg


def worst_error(got, want):
    return float(np.abs(got - want).max() / np.abs(want).max()) if len(want) else 0.0


def schedules(rep, rng, reqs):
    """r0 whole, r0 in drawn portions, and all requests in a drawn schedule of up to four live ones ({request: logits})."""
    toks = reqs["r0"]
    whole = rep.step({"step": 0, "entries": [{"id": "w", "tokens": toks, "want": list(range(len(toks)))}], "end": ["w"]})
    at, step, parts = 0, 0, []
    sizes = [rng.choice([2, 3, 5, 16, 17, 31]) for _ in range(4)] + [1] * len(toks)
    while at < len(toks):
        n = min(sizes[step], len(toks) - at)
        parts.append(rep.step({"step": step, "entries": [{"id": "c", "tokens": toks[at:at + n], "want": list(range(n))}],
                               "end": ["c"] if at + n == len(toks) else []}))
        at, step = at + n, step + 1
    waiting, live, at, got = list(reqs), [], {}, {k: [] for k in reqs}
    step = 0
    while waiting or live:
        while waiting and len(live) < 4 and rng.random() < 0.7:
            k = waiting.pop(0)
            live.append(k)
            at[k] = 0
        entries, end = [], []
        for k in list(live):
            if rng.random() < 0.25 and len(live) > 1:
                continue
            n = min(len(reqs[k]) - at[k], rng.choice([1, 1, 1, 2, 3, 7, 16, 17, 40]))
            entries.append({"id": k, "tokens": reqs[k][at[k]:at[k] + n], "want": list(range(n))})
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
                live.remove(k)
        if not entries:
            continue
        out, o = rep.step({"step": step, "entries": entries, "end": end}), 0
        for e in entries:
            got[e["id"]].append(out[o:o + len(e["tokens"])])
            o += len(e["tokens"])
        step += 1
    return whole, np.concatenate(parts), {k: np.concatenate(v) for k, v in got.items()}


@pytest.mark.parametrize("seed", range(10))
def test_drawn_configurations(seed, tmp_path):
    from ullm_amd.replay import Replayer
    rng = random.Random(7000 + seed)
    cfg = drawn_config(rng)
    w = plain.random_weights(cfg, seed)
    with open(os.path.join(tmp_path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(tmp_path, "model.safetensors"))
    wide = {k: v.double() for k, v in w.items()}
    reqs = {f"r{i}": [rng.randrange(cfg["vocab"]) for _ in range(rng.randint(20, 110))] for i in range(6)}
    want, sharp = {}, {}
    for k, t in reqs.items():
        plain.MARGINS = []
        want[k] = plain.forward(wide, cfg, t).float().numpy()
        # rows before the first token whose router nearly ties (32-bit sums may settle it otherwise, and every later
        # row sees that token through the states): only these are held to the 32-bit bound
        gaps = np.min([m.numpy() for m in plain.MARGINS], axis=0) if plain.MARGINS else np.full(len(t), np.inf)
        plain.MARGINS = None
        close_calls = np.nonzero(gaps < 1e-5)[0]
        sharp[k] = int(close_calls[0]) if len(close_calls) else len(t)
    assert sum(sharp.values()) >= 0.5 * sum(len(t) for t in reqs.values()), ("near-ties leave too few rows to compare", sharp)
    narrow = {k: v.float() for k, v in w.items()}
    plain.F = torch.float32
    try:
        # what 32-bit sums alone do to this model (four times that, as the engine sums in another order), at least 3e-5
        bound = {k: max(3e-5, 4 * worst_error(plain.forward(narrow, cfg, t).numpy()[:sharp[k]], want[k][:sharp[k]])) if sharp[k] else 1.0
                 for k, t in reqs.items()}
    finally:
        plain.F = torch.float64
    state = rng.getstate()
    whole, cut, mixed = schedules(Replayer(str(tmp_path), "float32", 512, 16, DEV, max_requests=4), rng, reqs)
    n0 = sharp["r0"]
    assert worst_error(whole[:n0], want["r0"][:n0]) <= bound["r0"], ("whole", worst_error(whole[:n0], want["r0"][:n0]), bound["r0"])
    assert worst_error(cut[:n0], want["r0"][:n0]) <= bound["r0"], ("cut", worst_error(cut[:n0], want["r0"][:n0]), bound["r0"])
    # a state element sees the same operations however the prompt is cut; a token's partial sums are added in an order
    # that goes by the step's shape
    assert worst_error(cut[:n0], whole[:n0]) <= 3e-6, ("whole and cut differ in 32-bit", worst_error(cut[:n0], whole[:n0]))
    for k in reqs:
        assert worst_error(mixed[k][:sharp[k]], want[k][:sharp[k]]) <= bound[k], (k, worst_error(mixed[k][:sharp[k]], want[k][:sharp[k]]), bound[k])
    # bfloat16: the same schedules.  What rounding does depends on the drawn model (up to twenty layer runs: a rounded
    # router input picks another expert at a close call, and then a row moves as a whole and the rows behind it a
    # little), so the bounds are multiples of what the plain implementation loses when nothing but its sublayers' inputs
    # are rounded to bfloat16: for the middle row and for 85 rows of 100.
    rng.setstate(state)
    rep = Replayer(str(tmp_path), "bfloat16", 512, 16, DEV, max_requests=4)
    whole, cut, mixed = schedules(rep, rng, reqs)
    for got, k in [(whole, "r0"), (cut, "r0")] + [(mixed[k], k) for k in reqs]:
        floor = np.abs(plain.forward(wide, cfg, reqs[k], round_to=torch.bfloat16).float().numpy() - want[k]).max(-1) / np.abs(want[k]).max()
        mid, most = 1e-2 + 4 * float(np.median(floor)), 2e-2 + 4 * float(np.quantile(floor, 0.85))
        err = np.abs(got - want[k]).max(-1) / np.abs(want[k]).max()
        assert np.median(err) <= mid and np.quantile(err, 0.85) <= most, (k, float(np.median(err)), float(np.quantile(err, 0.85)), mid, most)
