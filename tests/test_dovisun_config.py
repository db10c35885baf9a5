"""Dovisun without a GPU: the configuration reader, the plan it becomes (tensor names and shapes, the order the
layers run in with the passes' caches, the cache's groups), the stretched rotation table, and the plain
implementation's own pieces against each other."""
import copy
import math

import pytest
import torch

import plain_dovisun as plain
from ullm_amd.config import ConfigError, DovisunConfig
from ullm_amd.models import build_model
from ullm_amd.parts.position import Rotary


def attention(heads=6, kv=2, dim=8, vdim=12, scale=0.3, mlp=None):
    return dict(type="attention", mixer=dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale), mlp=mlp)


def latent(heads=3, dim=10, rot=6, vdim=14, q_rank=9, kv_rank=20, scale=0.2, base=5000.0, scaling=(4.0, 64, 8.0, 2.0), mlp=None):
    rot_cfg = dict(base=base, dims=rot)
    if scaling:
        rot_cfg["scaling"] = dict(factor=scaling[0], original=scaling[1], fast=scaling[2], slow=scaling[3])
    return dict(type="latent_attention", mixer=dict(heads=heads, dim=dim, rot_dim=rot, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank,
                                                    scale=scale, rot=rot_cfg), mlp=mlp)


DENSE = dict(kind="dense", ff=36)
MOE = dict(kind="moe", router=dict(experts=5, top=2), expert=dict(ff=10))
CFG = dict(architecture="Dovisun", vocab=70, width=24, norm=dict(eps=1e-4), embedding=dict(scale=2.0), logit_softcap=9.0,
           loop=dict(start=1, stop=3, times=3),
           layers=[attention(mlp=DENSE), latent(mlp=MOE), attention(heads=2, kv=2, dim=16, vdim=4, mlp=None), latent(mlp=DENSE)])


def test_the_plan_names_every_tensor_of_the_design_with_its_shape():
    cfg, model = build_model(CFG)
    assert isinstance(cfg, DovisunConfig) and cfg.num_hidden_layers == 4 and cfg.loops
    declared = {d.name: tuple(d.shape) for d in model.weight_decls()}
    assert declared == {k: tuple(v.shape) for k, v in plain.random_weights(CFG, 0).items()}


def test_layers_that_are_passed_again_keep_a_cache_per_pass():
    _, model = build_model(CFG)
    layers = [layer for layer, _ in model.run_order]
    mix = len(CFG["layers"])                                    # the step ahead of every pass stands behind the layers
    assert layers == [0, mix, 1, 2, mix, 1, 2, mix, 1, 2, 3]
    assert [i for i, first in plain.run_order(CFG)] == [i for i in layers if i != mix]
    assert [first for _, first in plain.run_order(CFG)] == [layers[n - 1] == mix for n, i in enumerate(layers) if i != mix]
    kept = [cache for layer, cache in model.run_order if layer != mix]
    assert len(set(kept)) == len(kept)                          # every run of a layer has a cache of its own
    groups, cache_group, states = model.cache_layout()
    assert not states
    held = sorted(n for g in groups for n, _ in g.layers)
    assert held == sorted(kept)
    # attention layers keep their key heads padded to a size the kernels take, latent layers one head [latent | rotated part]
    sizes = {(g.num_kv_heads, g.head_dim): len(g.layers) for g in groups}
    assert sizes == {(2, 32): 4, (1, 32): 4}


def test_no_loop_and_an_empty_loop():
    flat = copy.deepcopy(CFG)
    del flat["loop"]
    _, model = build_model(flat)
    assert model.run_order == [(i, i) for i in range(4)]
    assert "loop.in" not in {d.name for d in model.weight_decls()}
    empty = copy.deepcopy(CFG)
    empty["loop"] = dict(start=2, stop=2, times=5)
    _, model = build_model(empty)
    assert [layer for layer, _ in model.run_order] == [0, 1, 2, 3]
    assert [i for i, first in plain.run_order(empty)] == [0, 1, 2, 3] and not any(f for _, f in plain.run_order(empty))
    once = copy.deepcopy(CFG)
    once["loop"] = dict(start=0, stop=4, times=1)               # one pass: the embedding is still mixed in ahead of it
    _, model = build_model(once)
    assert [layer for layer, _ in model.run_order] == [4, 0, 1, 2, 3]
    assert plain.run_order(once)[0] == (0, True)


@pytest.mark.parametrize("dims,base,scaling", [(6, 5000.0, (4.0, 64, 8.0, 2.0)), (16, 1e6, (8.0, 512, 32.0, 1.0)),
                                               (32, 10000.0, (40.0, 4096, 32.0, 1.0)), (4, 100.0, (2.0, 16, 4.0, 0.5)),
                                               (8, 10000.0, None), (64, 500000.0, (1.0, 8192, 4.0, 1.0))])
def test_the_stretched_rotation_table(dims, base, scaling):
    rot = dict(dims=dims, base=base)
    if scaling:
        rot["scaling"] = dict(factor=scaling[0], original=scaling[1], fast=scaling[2], slow=scaling[3])
    freq, mag = plain.yarn_frequencies(rot)
    table = Rotary.make_table(dims, base, 300, scaling).double()
    pos = torch.arange(300, dtype=torch.float64)[:, None]
    assert (table[:, :dims // 2] - (pos * freq).cos() * mag).abs().max() < 1e-5
    assert (table[:, dims // 2:] - (pos * freq).sin() * mag).abs().max() < 1e-5
    if scaling:
        plain_freq = base ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims)
        # every pair turns between 1 / factor of its own frequency and its own frequency
        assert (freq <= plain_freq * (1 + 1e-12)).all() and (freq >= plain_freq / scaling[0] * (1 - 1e-12)).all()
        assert mag == pytest.approx(0.1 * math.log(scaling[0]) + 1.0)


def test_rotation_turns_pairs_half_a_head_apart():
    rot = dict(dims=4, base=100.0)
    x = torch.tensor([[1.0, 0.0, 0.0, 0.0, 7.0]], dtype=torch.float64).repeat(3, 1)
    out = plain.rotate_halves(x, torch.tensor([0, 1, 2]), rot)
    assert torch.allclose(out[0], x[0])
    # dim 0 pairs with dim 2 (frequency 1), dim 1 with dim 3; what lies behind ``dims`` passes
    assert torch.allclose(out[1], torch.tensor([math.cos(1.0), 0.0, math.sin(1.0), 0.0, 7.0], dtype=torch.float64))
    assert torch.allclose(out[2], torch.tensor([math.cos(2.0), 0.0, math.sin(2.0), 0.0, 7.0], dtype=torch.float64))


def test_softmax_with_one_more_term():
    s = torch.tensor([[0.5, -2.0, 3.0, -math.inf], [-50.0, -60.0, -55.0, -70.0], [80.0, 79.0, -math.inf, -math.inf]], dtype=torch.float64)
    p = plain.softmax_one_more(s)
    want = torch.exp(s) / (1 + torch.exp(s).sum(-1, keepdim=True))
    assert torch.allclose(p, want, rtol=1e-12, atol=0)
    assert p[1].sum() < 1e-20 and abs(float(p[2].sum()) - 1) < 1e-30 + 1e-12


def test_latent_attention_is_attention_over_up_projected_keys_and_values():
    """The plain latent attention, whose per-head keys are [W_uk c | one rotated part], against a direct form written
    with explicit loops over positions."""
    torch.manual_seed(3)
    m = latent()["mixer"]
    cfg = dict(CFG, layers=[latent()], loop=None)
    w = {k: v.double() for k, v in plain.random_weights(cfg, 5).items()}
    T, eps = 7, 1e-4
    h = torch.randn(T, 24, dtype=torch.float64)
    got = plain.latent_attention(w, "l0.mix", m, eps, h)
    H, d, r, dv, kr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    freq, mag = plain.yarn_frequencies(m["rot"])

    def turn(x, p):
        a = p * freq
        u, v = x[:r // 2], x[r // 2:]
        return torch.cat((u * a.cos() - v * a.sin(), v * a.cos() + u * a.sin())) * mag

    rows = []
    for t in range(T):
        cq = h[t] @ w["l0.mix.dq"].T
        cq = cq / torch.sqrt((cq * cq).mean() + eps) * w["l0.mix.dq.norm"]
        q = (w["l0.mix.uq"] @ cq).view(H, d + r)
        gate = torch.sigmoid(w["l0.mix.g"] @ h[t])
        heads = []
        for a in range(H):
            scores, values = [], []
            for j in range(t + 1):
                down = w["l0.mix.dkv"] @ h[j]
                c = down[:kr] / torch.sqrt((down[:kr] ** 2).mean() + eps) * w["l0.mix.dkv.norm"]
                key = torch.cat(((w["l0.mix.uk"] @ c).view(H, d)[a], turn(down[kr:], j)))
                qa = torch.cat((q[a, :d], turn(q[a, d:], t)))
                scores.append((qa @ key) * m["scale"])
                values.append((w["l0.mix.uv"] @ c).view(H, dv)[a])
            p = torch.softmax(torch.stack(scores), 0)
            heads.append((p[:, None] * torch.stack(values)).sum(0) * gate[a])
        rows.append(w["l0.mix.o"] @ torch.cat(heads))
    assert torch.allclose(got, torch.stack(rows), rtol=1e-9, atol=1e-12)


def test_routing_by_the_largest_logits():
    cfg = dict(CFG, layers=[attention(mlp=MOE)], loop=None)
    w = {k: v.double() for k, v in plain.random_weights(cfg, 6).items()}
    h = torch.randn(9, 24, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    ids, weights, z = plain.route(w, "l0.mlp", MOE, h)
    for t in range(9):
        order = sorted(range(5), key=lambda e: -float(z[t, e]))[:2]
        assert sorted(ids[t].tolist()) == sorted(order)
        e = torch.exp(z[t, ids[t]])
        assert torch.allclose(weights[t], e / e.sum())
    assert torch.allclose(z, h @ w["l0.mlp.router"].T + w["l0.mlp.router.b"])
    out = plain.experts(w, "l0.mlp", MOE, h)
    want = torch.stack([sum(weights[t, k] * plain.expert(w, f"l0.mlp.e{int(ids[t, k])}", h[t:t + 1])[0] for k in range(2)) for t in range(9)])
    assert torch.allclose(out, want)


def test_configurations_that_are_refused():
    for change, text in ((lambda c: c["layers"][0].update(type="conv"), "type"),
                         (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
                         (lambda c: c["layers"][0]["mixer"].update(kv_heads=4), "heads"),
                         (lambda c: c["layers"][1]["mixer"].update(rot_dim=5), "rot"),
                         (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=4), "rot.dims"),
                         (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].update(factor=0.0), "scaling"),
                         (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
                         (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "top"),
                         (lambda c: c["layers"][0]["mlp"].update(kind="experts"), "mlp"),
                         (lambda c: c["loop"].update(stop=5), "loop"), (lambda c: c["loop"].update(times=0), "loop"),
                         (lambda c: c["loop"].update(start=3, stop=2), "loop"),
                         (lambda c: c.pop("width"), "width"), (lambda c: c["norm"].pop("eps"), "eps"),
                         (lambda c: c.update(layers=[]), "layers")):
        bad = copy.deepcopy(CFG)
        change(bad)
        with pytest.raises(ConfigError, match=text):
            DovisunConfig.from_dict(bad)


def test_what_a_configuration_may_leave_out():
    lean = copy.deepcopy(CFG)
    del lean["embedding"], lean["logit_softcap"], lean["loop"]
    del lean["layers"][1]["mixer"]["rot"]["scaling"]
    cfg = DovisunConfig.from_dict(lean)
    assert cfg.embedding_scale == 1.0 and cfg.logit_softcap == 0.0 and not cfg.loops and not cfg.has_loop
    assert cfg.layers[1].mixer.rot_scaling is None


def test_the_named_size_for_random_weights():
    from ullm_amd.config import parse_random_weights
    d, seed = parse_random_weights("dovisun-2048:5")
    cfg, model = build_model(d)
    assert seed == 5 and isinstance(cfg, DovisunConfig) and cfg.loops and len(model.run_order) == 6 + 2 + 2
