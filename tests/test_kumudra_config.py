"""Kumudra without a GPU: the configuration reader and what it refuses, the plan it becomes (tensor names and shapes,
the order the layers run in with the passes' caches and state, what a block of two mixers keeps), the rotation table
stretched by wavelength against the formula, and the plain implementation's own pieces against explicit loops."""
import copy
import math

import pytest
import torch

import plain_kumudra as plain
from ullm_amd.config import ConfigError, KumudraConfig
from ullm_amd.models import build_model
from ullm_amd.parts import KVNeed, StateNeed, cache_needs_of
from ullm_amd.parts.position import Rotary


def gla(heads=3, dim=8, vdim=12, tau=4.0, mlp=None):
    return dict(type="gla", mixer=dict(heads=heads, dim=dim, vdim=vdim, tau=tau, rank=5), mlp=mlp)


def lightning(heads=2, dim=12, vdim=4, decay=(0.5, 0.97), mlp=None):
    return dict(type="lightning", mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay)), mlp=mlp)


def parallel(heads=6, kv=2, dim=8, vdim=12, window=9, rot=4, scaling=(4.0, 1.0, 4.0, 64), mlp=None):
    rot_cfg = dict(base=500.0, dims=rot)
    if scaling:
        rot_cfg["scaling"] = dict(factor=scaling[0], low=scaling[1], high=scaling[2], original=scaling[3])
    left = dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=0.3, mask=dict(size=window), rot=rot_cfg)
    return dict(type="parallel", mixer=dict(left=left, right=dict(heads=5, dim=4, rank=3), left_scale=0.7, right_scale=1.2), mlp=mlp)


DENSE = dict(kind="dense", ff=36)
MOE = dict(kind="moe", router=dict(experts=5, top=2, scale=2.5), expert=dict(ff=10))
CFG = dict(architecture="Kumudra", vocab=70, width=24, norm=dict(eps=1e-4), embedding=dict(scale=2.0), residual_mult=0.5,
           streams=3, loop=dict(start=1, stop=3, times=3),
           layers=[gla(mlp=DENSE), lightning(mlp=MOE), parallel(mlp=None), gla(heads=1, dim=4, vdim=4, mlp=MOE)])


def test_the_plan_names_every_tensor_of_the_design_with_its_shape():
    cfg, model = build_model(CFG)
    assert isinstance(cfg, KumudraConfig) and cfg.num_hidden_layers == 4 and cfg.streams == 3
    declared = {d.name: tuple(d.shape) for d in model.weight_decls() if d.alias_of is None}
    assert declared == plain.tensor_shapes(CFG)
    tied = [d for d in model.weight_decls() if d.alias_of is not None]
    assert [(d.name, d.alias_of) for d in tied] == [("head", "embed")]


def test_layers_that_are_passed_again_keep_caches_and_state_per_pass():
    cfg, model = build_model(CFG)
    layers = [layer for layer, _ in model.run_order]
    assert layers == [0, 1, 2, 1, 2, 1, 2, 3] == plain.run_order(CFG) == cfg.run_order()
    kept = [cache for _, cache in model.run_order]
    assert len(set(kept)) == len(kept)
    groups, cache_group, states = model.cache_layout()
    # the softmax half of every run of layer 2 keeps keys and values in pages, heads stored at a size the kernels take
    assert len(groups) == 1 and (groups[0].num_kv_heads, groups[0].head_dim, groups[0].window) == (2, 32, 9)
    assert len(groups[0].layers) == 3
    # every run keeps state: the heads' matrices, and for time mixing the last input row ahead of them
    sizes = sorted(need.shape[0] for need in states.values())
    assert sizes == sorted([3 * 8 * 12] + [2 * 12 * 4] * 3 + [24 + 5 * 4 * 4] * 3 + [16])
    assert all(need.dtype == torch.float32 and need.graph_safe for need in states.values())


def test_a_block_of_two_mixers_keeps_pages_and_state():
    _, model = build_model(CFG)
    needs = cache_needs_of(model.blocks[2])
    assert [type(n) for n in needs] == [KVNeed, StateNeed]
    assert cache_needs_of(model.blocks[0])[0].shape == (3 * 8 * 12,)


def test_no_loop_one_pass_one_stream_and_defaults():
    c = copy.deepcopy(CFG)
    del c["loop"]
    _, model = build_model(c)
    assert model.run_order == [(i, i) for i in range(4)]
    c["loop"] = dict(start=2, stop=2, times=5)
    assert [l for l, _ in build_model(c)[1].run_order] == [0, 1, 2, 3]
    c["loop"] = dict(start=0, stop=4, times=1)
    assert [l for l, _ in build_model(c)[1].run_order] == [0, 1, 2, 3]
    c["streams"] = 1
    del c["residual_mult"], c["embedding"]
    cfg, model = build_model(c)
    assert cfg.residual_mult == 1.0 and cfg.embedding_scale == 1.0 and model.plan.streams == 1
    # with one copy a checkpoint may leave the coefficients out: they are declared with ones to fall back on
    assert all(d.default == 1.0 for d in model.weight_decls() if ".hc" in d.name)
    c["streams"] = 3
    assert all(d.default is None for d in build_model(c)[1].weight_decls() if ".hc" in d.name)


@pytest.mark.parametrize("change,text", [
    (lambda c: c["layers"][0].update(type="mamba"), "type"),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][2]["mixer"]["left"].update(kv_heads=4), "kv heads"),
    (lambda c: c["layers"][2]["mixer"]["left"]["rot"].update(dims=3), "rot.dims"),
    (lambda c: c["layers"][2]["mixer"].pop("right"), "right"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "top"),
    (lambda c: c["layers"][0]["mlp"].update(kind="glu"), "mlp.kind"),
    (lambda c: c["loop"].update(stop=5), "loop"),
    (lambda c: c.update(streams=0), "streams"),
    (lambda c: c["layers"][0]["mixer"].update(tau=0.0), "tau"),
    (lambda c: c.pop("width"), "width"),
])
def test_what_the_reader_refuses(change, text):
    c = copy.deepcopy(CFG)
    change(c)
    with pytest.raises(ConfigError, match=text):
        build_model(c)


@pytest.mark.parametrize("dims,base,scaling", [(8, 10000.0, (8.0, 1.0, 4.0, 64)), (16, 500.0, (4.0, 2.0, 8.0, 200)),
                                               (4, 50.0, (2.0, 1.0, 2.0, 16)), (6, 1000.0, None)])
def test_the_rotation_table_stretched_by_wavelength(dims, base, scaling):
    rows = 40
    table = Rotary.make_table(dims, base, rows, None if scaling is None else ("by_wavelength",) + scaling)
    assert table.shape == (rows, dims) and table.dtype == torch.float32
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling is not None:
            factor, low, high, original = scaling
            wavelength = 2 * math.pi / f
            if wavelength > original / low:
                f /= factor
            elif wavelength >= original / high:
                s = (original / wavelength - low) / (high - low)
                f = (1 - s) * f / factor + s * f
        for p in (0, 1, 7, rows - 1):
            assert abs(float(table[p, i]) - math.cos(p * f)) < 1e-6 and abs(float(table[p, dims // 2 + i]) - math.sin(p * f)) < 1e-6
    assert torch.allclose(plain.rotary_frequencies(dims, base, scaling).float(),
                          torch.atan2(table[1, dims // 2:], table[1, :dims // 2]).float(), atol=1e-6)


def test_the_stretch_has_all_three_ranges_in_one_table():
    f = plain.rotary_frequencies(16, 500.0, (4.0, 1.0, 4.0, 64))
    plain_f = plain.rotary_frequencies(16, 500.0, None)
    ratio = (f / plain_f).tolist()
    assert ratio[0] == 1.0 and abs(ratio[-1] - 0.25) < 1e-12 and any(0.25 < r < 1.0 for r in ratio)


def test_the_plain_recurrence_against_its_sums():
    """o_t after the update is sum_j (prod_{j < i <= t} d_i) (q_t . k_j ...) per channel; with a bonus the current token
    enters with the bonus instead of a decay and the state it sees is the one before."""
    g = torch.Generator().manual_seed(0)
    T, H, d, dv = 7, 2, 3, 4
    q, k = torch.randn(T, H, d, generator=g, dtype=plain.F), torch.randn(T, H, d, generator=g, dtype=plain.F)
    v = torch.randn(T, H, dv, generator=g, dtype=plain.F)
    dec = torch.rand(T, H, d, generator=g, dtype=plain.F)
    u = torch.randn(H, d, generator=g, dtype=plain.F)
    after, before = plain.decayed_state_outputs(q, k, v, dec), plain.decayed_state_outputs(q, k, v, dec, bonus=u)
    for t in range(T):
        for h in range(H):
            want_a, want_b = torch.zeros(dv, dtype=plain.F), torch.zeros(dv, dtype=plain.F)
            for j in range(t + 1):
                carried = torch.ones(d, dtype=plain.F)
                for i in range(j + 1, t + 1):
                    carried = carried * dec[i, h]
                want_a += (q[t, h] * carried * k[j, h]).sum() * v[j, h]
                if j < t:
                    kept = torch.ones(d, dtype=plain.F)
                    for i in range(j + 1, t):
                        kept = kept * dec[i, h]
                    want_b += (q[t, h] * kept * k[j, h]).sum() * v[j, h]
                else:
                    want_b += (q[t, h] * u[h] * k[j, h]).sum() * v[j, h]
            assert torch.allclose(after[t, h], want_a, atol=1e-12) and torch.allclose(before[t, h], want_b, atol=1e-12)


def test_the_plain_streams_against_a_loop():
    g = torch.Generator().manual_seed(1)
    S, T, W = 3, 4, 5
    xs = torch.randn(S, T, W, generator=g, dtype=plain.F)
    w = {"p.hc1.in": torch.randn(S, generator=g, dtype=plain.F), "p.hc1.out": torch.randn(S, generator=g, dtype=plain.F),
         "p.hc1.mix": torch.randn(S, S, generator=g, dtype=plain.F)}
    got = plain.hyper_sublayer(xs, lambda u: 2.0 * u, w, "p", 1, 0.5)
    for t in range(S):
        u = sum(w["p.hc1.in"][s] * xs[s] for s in range(S))
        want = sum(w["p.hc1.mix"][s, t] * xs[s] for s in range(S)) + 0.5 * w["p.hc1.out"][t] * 2.0 * u
        assert torch.allclose(got[t], want, atol=1e-12)


def test_the_plain_router_weights_and_window():
    g = torch.Generator().manual_seed(2)
    h = torch.randn(6, 8, generator=g, dtype=plain.F)
    w = {"m.router": torch.randn(4, 8, generator=g, dtype=plain.F), "m.correction": torch.tensor([0.0, 5.0, 0.0, -5.0], dtype=plain.F)}
    for e in range(4):
        w.update({f"m.e{e}.gate": torch.randn(3, 8, generator=g, dtype=plain.F), f"m.e{e}.up": torch.randn(3, 8, generator=g, dtype=plain.F),
                  f"m.e{e}.down": torch.randn(8, 3, generator=g, dtype=plain.F)})
    f = dict(kind="moe", router=dict(experts=4, top=2, scale=3.0), expert=dict(ff=3))
    got = plain.routed_ff(h, w, "m", f)
    s = torch.sigmoid(h @ w["m.router"].T)
    for t in range(6):
        # the correction decides the choice (expert 1 always, expert 3 never) and stays out of the weights
        other = 0 if s[t, 0] >= s[t, 2] else 2
        total = s[t, 1] + s[t, other]
        want = sum(3.0 * s[t, e] / total * plain.gated_unit(h[t], w[f"m.e{e}.gate"], w[f"m.e{e}.up"], w[f"m.e{e}.down"]) for e in (1, other))
        assert torch.allclose(got[t], want, atol=1e-12)


def test_a_file_may_hold_the_tensors_of_a_feed_forward_that_a_layer_does_not_have():
    from ullm_amd.weights.loader import WeightError, check_against
    _, model = build_model(CFG)
    index = {d.name: ("f", tuple(d.shape), "BF16") for d in model.weight_decls() if d.alias_of is None}
    extra = {"l2.norm2": ("f", (24,), "BF16"), "l2.hc2.mix": ("f", (3, 3), "BF16")}
    check_against(model.weight_decls(), {**index, **extra}, frozenset(model.plan.unused_tensors))
    with pytest.raises(WeightError, match="unexpected"):
        check_against(model.weight_decls(), {**index, "l0.hc3.in": ("f", (3,), "BF16")}, frozenset(model.plan.unused_tensors))
