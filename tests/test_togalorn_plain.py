"""Togalorn without a GPU: the configuration through its file and back, errors that name the key, the model as data
(names, shapes, run order, what each call caches), and the plain implementation's own mechanisms."""
import json
import math
import os

import pytest
import torch

import plain_togalorn as P
from tiny_togalorn import CONFIGS, TG_A, TG_B, TG_D, write_tiny

from gesso_amd.config import TogalornConfig, load_config
from gesso_amd.errors import ConfigError


def gen(seed):
    return torch.Generator().manual_seed(seed)


# ------------------------------------------------------------------ configuration

@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_configuration_through_its_file_and_back(name, tmp_path):
    cfg, _ = CONFIGS[name]
    raw = cfg.to_json()
    assert TogalornConfig.from_dict(json.loads(json.dumps(raw))) == cfg
    d = tmp_path / "m"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(raw))
    arch, back = load_config(str(d))
    assert arch.name == "Togalorn" and back == cfg


def test_keys_left_out_take_their_defaults_and_unknown_keys_name_themselves():
    raw = TG_A.to_json()
    for key in ("canon", "loop", "embedding"):
        del raw[key]
    del raw["norm"]["groups"]
    raw["layers"][0]["mlp"]["router"].pop("identity")
    cfg = TogalornConfig.from_dict(raw)
    assert cfg.canon_taps is None and cfg.loop is None and cfg.embedding_scale == 1.0 and cfg.norm_groups == 1
    assert cfg.layers[0].mlp.identity == 0
    for path, where in ((("window",), "config.json"), (("layers", 0, "mixer", "chunk"), "layers[0].mixer"),
                        (("layers", 1, "mixer", "rot", "scaling"), "layers[1].mixer.rot"),
                        (("layers", 0, "mlp", "router", "bias"), "layers[0].mlp.router")):
        raw = TG_A.to_json()
        at = raw
        for k in path[:-1]:
            at = at[k]
        at[path[-1]] = 3
        with pytest.raises(ConfigError) as err:
            TogalornConfig.from_dict(raw)
        assert path[-1] in str(err.value) and where in str(err.value)


@pytest.mark.parametrize("change,word", [
    (lambda r: r["layers"][0].__setitem__("type", "attention"), "type"),
    (lambda r: r["layers"][1]["mixer"]["rot"].__setitem__("dims", 8), "rot.dims"),
    (lambda r: r["loop"].__setitem__("stop", 9), "loop"),
    (lambda r: r["norm"].__setitem__("groups", 5), "groups"),
    (lambda r: r["layers"][0]["mixer"].__setitem__("groups", 3), "groups"),
    (lambda r: r["layers"][0]["mlp"]["router"].__setitem__("top", 9), "top"),
    (lambda r: r["layers"][0]["mlp"].__setitem__("kind", "dense"), "kind"),
    (lambda r: r["layers"][0]["mixer"].pop("state"), "state")])
def test_contradictions_are_errors(change, word):
    raw = TG_A.to_json()
    change(raw)
    with pytest.raises(ConfigError) as err:
        TogalornConfig.from_dict(raw)
    assert word in str(err.value)


# ------------------------------------------------------------------ the model as data

def test_run_order_names_and_caches():
    from gesso_amd.config.registry import architecture_of
    from gesso_amd.models.model import tensor_table
    from gesso_amd.parts import PagedKV, SlotState, part_class
    spec = architecture_of(TG_B.to_json()).to_spec(TG_B)
    assert [c.layer for c in spec.schedule] == [0, 1, 2, 1, 2, 3] and spec.reentry.at == (1, 3)
    assert [c.layer for c in architecture_of(TG_A.to_json()).to_spec(TG_A).schedule] == [0, 1, 2, 0, 1, 2, 3]
    d = architecture_of(TG_D.to_json()).to_spec(TG_D)
    assert [c.layer for c in d.schedule] == [0, 1, 2] and d.reentry.at == (0,)
    table = tensor_table(spec)
    assert table["loop.in"].shape == (64, 128) and table["loop.step"].shape == (2, 64)
    assert table["l1.canon1"].shape == (64, 2) and table["l0.mix.g"].shape == (2 * 24, 64)
    assert table["l2.mix.in"].shape == (2 * 24 + 2 * 2 * 8 + 2, 64) and table["l2.mix.conv"].shape == (24 + 2 * 2 * 8, 5)
    assert table["l3.mlp.router"].shape == (4, 64) and "l3.mlp.e2.gate" not in table and "l3.mlp.e1.down" in table
    assert "l0.mlp.router" not in table and "l1.mlp.shared.up" not in table and table["l3.mlp.shared.down"].shape == (64, 40)
    assert "l0.norm2" not in table
    needs = [part_class("block", spec.blocks[c.layer]).cache_need(spec.blocks[c.layer]) for c in spec.schedule]
    # every call keeps the history of its input convolution beside what its mixer keeps
    assert all(isinstance(n, tuple) and isinstance(n[0], SlotState) for n in needs)
    assert needs[0][1] == PagedKV(1, 32 + 16, None, value_dim=0) and needs[1][1] == PagedKV(1, 36 + 8, None, value_dim=0)
    names = [[e[0] for e in n[1].entries()] for n in needs if isinstance(n[1], SlotState)]
    assert names == [["conv_history", "state"]] * 3
    # the two passes' attention calls lie in one page group as two members
    from gesso_amd.cache.manager import CacheLayout
    layout = CacheLayout.plan(needs, [None] * len(needs))
    assert sorted(len(g.members) for g in layout.paged) == [1, 2]
    assert len(layout.slots) == 6 + 3


# ------------------------------------------------------------------ the plain implementation's mechanisms

def test_norm_in_parts():
    x = torch.randn(5, 12, generator=gen(1), dtype=torch.float64)
    w = torch.randn(12, generator=gen(2), dtype=torch.float64)
    got = P.group_norm(x, w, 1e-6, 3)
    for g in range(3):
        part = x[:, 4 * g:4 * g + 4]
        want = part / torch.sqrt((part ** 2).mean(-1, keepdim=True) + 1e-6) * w[4 * g:4 * g + 4]
        assert torch.allclose(got[:, 4 * g:4 * g + 4], want)
    # scaling one part leaves the others alone; one part is the plain norm
    y = x.clone()
    y[:, :4] *= 100.0
    assert torch.allclose(P.group_norm(y, w, 1e-6, 3)[:, 4:], got[:, 4:])
    assert torch.allclose(P.group_norm(x, w, 1e-6, 1), P.rms(x, 1e-6) * w)


def test_convolution_by_hand_and_its_first_tokens():
    x = torch.tensor([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0], [4.0, 40.0]], dtype=torch.float64)
    taps = torch.tensor([[0.5, 0.0, 2.0], [1.0, -1.0, 0.0]], dtype=torch.float64)      # the last column meets the newest
    got = P.causal_conv(x, taps)
    want = torch.tensor([[2.0, 0.0], [4.0, -10.0], [6.5, -10.0], [9.0, -10.0]], dtype=torch.float64)
    assert torch.equal(got, want)
    assert torch.equal(P.causal_conv(x, taps, torch.tensor([1.0, 2.0], dtype=torch.float64)), want + torch.tensor([1.0, 2.0]))
    one = torch.tensor([[3.0], [0.5]], dtype=torch.float64)
    assert torch.equal(P.causal_conv(x, one), x * one[:, 0])


def test_rotation_pairs_neighbours_and_scores_depend_on_distance_alone():
    x = torch.zeros(1, 6, dtype=torch.float64)
    x[0, 2] = 1.0
    y = P.rotate_interleaved(x, [3], 100.0, 4)                                   # pair (2, 3) turns by 3 * 100^(-2/4)
    a = 3 * 100.0 ** -0.5
    assert torch.allclose(y[0], torch.tensor([0, 0, math.cos(a), math.sin(a), 0, 0], dtype=torch.float64))
    q = torch.randn(1, 8, generator=gen(3), dtype=torch.float64)
    k = torch.randn(1, 8, generator=gen(4), dtype=torch.float64)
    s = [float(P.rotate_interleaved(q, [i], 1e4, 8)[0] @ P.rotate_interleaved(k, [j], 1e4, 8)[0]) for i, j in ((9, 4), (105, 100), (5, 0))]
    assert s[0] == pytest.approx(s[1], abs=1e-12) and s[0] == pytest.approx(s[2], abs=1e-12)
    assert torch.equal(P.rotate_interleaved(q, [0], 1e4, 8), q)


def test_state_space_against_the_explicit_sum_over_the_past():
    T, H, Pd, G, N = 9, 4, 3, 2, 5
    g = gen(5)
    x, B, C = (torch.randn(s, generator=g, dtype=torch.float64) for s in ((T, H, Pd), (T, G, N), (T, G, N)))
    dt = torch.rand(T, H, generator=g, dtype=torch.float64) + 0.1
    a_log = torch.tensor([-30.0, -1.0, 0.0, 1.0], dtype=torch.float64)           # the first head hardly forgets
    d = torch.randn(H, generator=g, dtype=torch.float64)
    y = P.state_space(x, B, C, dt, a_log, d, H // G)
    for h in range(H):
        grp = h // (H // G)
        for t in range(T):
            want = d[h] * x[t, h]
            for s in range(t + 1):
                keep = math.exp(-math.exp(float(a_log[h])) * float(dt[s + 1:t + 1, h].sum()))
                want = want + keep * dt[s, h] * (C[t, grp] @ B[s, grp]) * x[s, h]
            assert torch.allclose(y[t, h], want, atol=1e-10)
    # heads of one group share B and C, heads of different groups do not
    B2 = B.clone()
    B2[:, 1] += 1.0
    y2 = P.state_space(x, B2, C, dt, a_log, d, H // G)
    assert torch.equal(y2[:, :2], y[:, :2]) and not torch.allclose(y2[:, 2:], y[:, 2:])


def test_router_choice_weights_correction_and_identity_experts():
    h = torch.eye(4, dtype=torch.float64)
    router = torch.tensor([[2.0, 0, 0, 0], [1.0, 3, 0, 0], [0.5, 0, 1, 0], [0.0, 1, 2, 0.5]], dtype=torch.float64)
    zero = torch.zeros(4, dtype=torch.float64)
    chosen, weights, s = P.route(h, router, zero, 2)
    assert chosen[0].tolist() == [0, 1] and torch.allclose(weights.sum(-1), torch.ones(4, dtype=torch.float64))
    assert torch.allclose(weights[0], s[0, :2] / s[0, :2].sum())
    # equal scores: the lowest index first
    assert chosen[3].tolist()[0] == 3 and P.route(h[3:], torch.zeros(4, 4, dtype=torch.float64), zero, 2)[0][0].tolist() == [0, 1]
    # the correction changes the choice, not the weights' source
    corr = torch.tensor([0.0, 0.0, 0.0, 5.0], dtype=torch.float64)
    chosen2, weights2, _ = P.route(h, router, corr, 2)
    assert chosen2[0].tolist() == [3, 0] and torch.allclose(weights2[0], s[0, [3, 0]] / s[0, [3, 0]].sum())
    # an identity expert gives back its input, weighted
    W = 4
    w = {"m.router": router, "m.correction": corr, "m.e0.gate": torch.zeros(3, W, dtype=torch.float64),
         "m.e0.up": torch.zeros(3, W, dtype=torch.float64), "m.e0.down": torch.ones(W, 3, dtype=torch.float64)}
    for e in (1, 2):
        for k in ("gate", "up", "down"):
            w[f"m.e{e}.{k}"] = w[f"m.e0.{k}"]
    m = {"router": {"experts": 3, "top": 2, "identity": 1}, "expert": {"ff": 3, "limit": 1.0}, "shared": None}
    x = torch.randn(1, W, generator=gen(6), dtype=torch.float64)
    chosen3, weights3, _ = P.route(x, router, corr, 2)
    assert chosen3[0, 0] == 3
    assert torch.allclose(P.moe(x, w, "m", m), weights3[0, 0] * x)               # experts with zero gate put out nothing


def test_expert_limits():
    gate = torch.tensor([[1.0]], dtype=torch.float64)
    up = torch.tensor([[1.0]], dtype=torch.float64)
    down = torch.tensor([[1.0]], dtype=torch.float64)
    f = lambda v, lim: float(P.expert(torch.tensor([[v]], dtype=torch.float64), gate, up, down, lim))
    sig = lambda z: 1 / (1 + math.exp(-z))
    assert f(0.5, 1.0) == pytest.approx(0.5 * sig(1.702 * 0.5) * 1.5)
    assert f(3.0, 1.0) == pytest.approx(1.0 * sig(1.702) * 2.0)                  # both cut from above
    assert f(-3.0, 1.0) == pytest.approx(-3.0 * sig(-1.702 * 3.0) * 0.0, abs=1e-12)   # the gate is not cut from below, up is
    assert f(-3.0, 5.0) == pytest.approx(-3.0 * sig(-1.702 * 3.0) * -2.0)


def test_attention_finds_a_key_far_back_and_never_one_ahead():
    m = {"heads": 2, "dim": 4, "rot_dim": 4, "vdim": 3, "kv_rank": 6, "q_rank": 5, "scale": 0.3, "rot": {"base": 1e4, "dims": 4}}
    W, T = 8, 40
    g = gen(7)
    shapes = {"dq": (5, W), "dq.norm": (5,), "uq": (16, 5), "dkv": (10, W), "dkv.norm": (6,), "uk": (8, 6), "uv": (6, 6),
              "g": (6, W), "o": (W, 6)}
    w = {"m." + k: torch.randn(s, generator=g, dtype=torch.float64) * 0.5 for k, s in shapes.items()}
    h = torch.randn(T, W, generator=g, dtype=torch.float64)
    base = P.latent_attention(h, w, "m", m, 1e-6, list(range(T)))
    h2 = h.clone()
    h2[30] += 1.0
    moved = P.latent_attention(h2, w, "m", m, 1e-6, list(range(T)))
    assert torch.equal(moved[:30], base[:30]) and not torch.allclose(moved[39], base[39])
    h3 = h.clone()
    h3[0] *= 3.0
    assert not torch.allclose(P.latent_attention(h3, w, "m", m, 1e-6, list(range(T)))[39], base[39])


def test_a_layer_by_hand_and_the_loop(tmp_path):
    d = write_tiny(str(tmp_path), "B")
    cfg, w = P.read_config(d), P.read_weights(d)
    ids = [5, 17, 3, 99, 41, 8, 120]
    outs = []
    logits = P.forward(cfg, w, ids, layers_out=outs)
    assert len(outs) == 6 and logits.shape == (7, 150)
    pos = list(range(7))
    x0 = P.embedding(w["embed"], ids, 1.0)
    a = P.group_norm(x0, w["l0.norm1"], 1e-5, 1)
    x1 = x0 + P.latent_attention(a + P.causal_conv(a, w["l0.canon1"]), w, "l0.mix", cfg["layers"][0]["mixer"], 1e-5, pos)
    assert torch.allclose(outs[0], x1)
    x = torch.cat([x1, x0], 1) @ w["loop.in"].T + w["loop.step"][0]
    x = P.layer(P.layer(x, w, 1, cfg, pos), w, 2, cfg, pos)
    assert torch.allclose(outs[2], x)
    x = torch.cat([x, x0], 1) @ w["loop.in"].T + w["loop.step"][1]
    assert torch.allclose(outs[3], P.layer(x, w, 1, cfg, pos))
    # a token's logits do not depend on what follows it
    assert torch.allclose(P.forward(cfg, w, ids[:4]), logits[:4])
    assert P.greedy(cfg, w, ids, 2)[:7] == ids
