"""Penasun without a GPU: its configuration (every size from the file, defaults for what a layer
leaves out, errors that name the key), the tensors its parts ask for, the size of the state a
sequence carries, and the plain implementation against itself (a prompt at once equals the same
tokens one by one, through what it carries)."""
import copy

import pytest
import torch

import hector_engine_amd  # noqa: F401
from hector_engine_amd.config.base import ConfigError
from hector_engine_amd.parts.base import BuildEnv
from hector_engine_amd.registry import build_model, config_from_dict
from tests.plain import penasun_plain as P


def scan(heads, vdim, state, groups=1, conv=4, norm_groups=1):
    return {"conv": conv, "groups": groups, "heads": heads, "norm_groups": norm_groups, "state": state, "vdim": vdim}


def attn(heads, kv, dim, vdim, scale, diff, q_temp=None):
    m = {"diff": diff, "dim": dim, "heads": heads, "kv_heads": kv, "scale": scale, "vdim": vdim}
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return m


def moe(experts, identity, top, ff, limit, count=1, keep=1, scale=1.0):
    return {"expert": {"ff": ff, "limit": limit}, "kind": "moe",
            "router": {"experts": experts, "groups": {"count": count, "keep": keep}, "identity": identity,
                       "scale": scale, "top": top}}


def layer(kind, mixer, mlp=None):
    return {"mixer": mixer, "mlp": mlp, "type": kind}


SMALL = {"architecture": "Penasun", "vocab": 61, "width": 24, "norm": {"eps": 1e-6},
         "layers": [layer("attention", attn(4, 2, 8, 16, 0.3, 0.4, (0.5, 3)), moe(4, 2, 2, 16, 1.5, 3, 2, 1.5)),
                    layer("mamba2", scan(3, 8, 12, 1, 3, 3)),
                    layer("mamba2", scan(2, 4, 80, 2, 2, 1), moe(3, 0, 1, 8, 0.5))]}


def test_configuration_reads_back_and_every_size_comes_from_the_file():
    cfg = config_from_dict(copy.deepcopy(SMALL))
    assert cfg.to_dict() == SMALL
    assert [l.type for l in cfg.layers] == ["attention", "mamba2", "mamba2"]
    a, s = cfg.layers[0].mixer, cfg.layers[2].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.diff, a.q_temp_coef, a.q_temp_every) == (4, 2, 8, 16, 0.3, 0.4, 0.5, 3)
    assert (s.heads, s.vdim, s.state, s.groups, s.conv, s.norm_groups) == (2, 4, 80, 2, 2, 1)
    f = cfg.layers[0].mlp
    assert (f.experts, f.identity, f.top, f.ff, f.limit, f.group_count, f.group_keep, f.scale) == (4, 2, 2, 16, 1.5, 3, 2, 1.5)
    assert cfg.layers[1].mlp is None


def test_defaults_for_what_a_layer_leaves_out():
    d = copy.deepcopy(SMALL)
    del d["layers"][0]["mixer"]["q_temp"], d["layers"][0]["mixer"]["kv_heads"], d["layers"][0]["mixer"]["vdim"]
    del d["layers"][2]["mlp"]["router"]["groups"], d["layers"][2]["mlp"]["router"]["identity"]
    del d["layers"][1]["mixer"]["groups"], d["layers"][1]["mixer"]["norm_groups"]
    cfg = config_from_dict(d)
    a = cfg.layers[0].mixer
    assert (a.kv_heads, a.vdim, a.q_temp_every) == (4, 8, 0)
    assert (cfg.layers[2].mlp.group_count, cfg.layers[2].mlp.group_keep, cfg.layers[2].mlp.identity) == (1, 1, 0)
    assert (cfg.layers[1].mixer.groups, cfg.layers[1].mixer.norm_groups) == (1, 1)


@pytest.mark.parametrize("path,value,word", [
    (("layers", 0, "type"), "conv", "unknown mixer type"),
    (("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"),
    (("layers", 1, "mixer", "groups"), 2, "groups"),
    (("layers", 1, "mixer", "norm_groups"), 5, "norm_groups"),
    (("layers", 0, "mlp", "router", "groups", "count"), 4, "groups.count"),
    (("layers", 0, "mlp", "router", "top"), 5, "router.top"),
    (("layers", 0, "mlp", "kind"), "dense", "unknown kind"),
    (("layers", 0, "mixer", "q_temp", "every"), 0, "q_temp.every"),
    (("width",), 0, "width"),
])
def test_errors_name_the_key(path, value, word):
    d = copy.deepcopy(SMALL)
    at = d
    for k in path[:-1]:
        at = at[k]
    at[path[-1]] = value
    with pytest.raises(ConfigError, match=word):
        config_from_dict(d)


def test_tensors_the_parts_ask_for_and_the_state_a_sequence_carries():
    model = build_model(config_from_dict(copy.deepcopy(SMALL)), BuildEnv(torch.device("cpu"), torch.float32))
    specs = {k: tuple(v.shape) for k, v in model.tensor_specs().items()}
    assert specs["embed"] == (61, 24) and specs["final.norm"] == (24,) and specs["l1.norm1"] == (24,)
    assert "l1.norm2" not in specs and "head" not in specs
    assert specs["l0.mix.q"] == (4 * 2 * 8, 24) and specs["l0.mix.k"] == (2 * 2 * 8, 24) and specs["l0.mix.v"] == (2 * 16, 24)
    assert specs["l0.mix.q.b"] == (64,) and specs["l0.mix.o"] == (24, 64) and specs["l0.mix.o.b"] == (24,)
    assert all(specs[f"l0.mix.{n}"] == (8,) for n in ("lq1", "lk1", "lq2", "lk2"))
    assert specs["l0.mlp.router"] == (6, 24) and specs["l0.mlp.correction"] == (6,)
    assert specs["l0.mlp.e3.gate"] == (16, 24) and specs["l0.mlp.e3.down"] == (24, 16) and "l0.mlp.e4.gate" not in specs
    inner, bc = 3 * 8, 2 * 1 * 12
    assert specs["l1.mix.in"] == (2 * inner + bc + 3, 24) and specs["l1.mix.conv"] == (inner + bc, 3)
    assert specs["l1.mix.conv.b"] == (inner + bc,) and specs["l1.mix.norm"] == (inner,) and specs["l1.mix.o"] == (24, inner)
    assert specs["l1.mix.dt_bias"] == specs["l1.mix.A_log"] == specs["l1.mix.D"] == (3,)
    plans = model.run_plans()
    # two carried inputs of 48 channels, then 3 x 8 x 16 floats of state (12 state dims in two shares of 8)
    assert plans[0].state_bytes == 0 and plans[1].state_bytes == 4 * (2 * 48 + 3 * 8 * 16)
    # one carried input of 8 + 2 * 2 * 80 channels, then 2 x 4 x 128 floats (80 dims in sixteen shares of 8)
    assert plans[2].state_bytes == 4 * 328 + 4 * 2 * 4 * 128
    # a differential attention keeps two keys a kv head, and the values once a map
    assert plans[0].kv.kv_heads == 4 and plans[1].kv is None


def random_weights(cfg_dict, seed):
    model = build_model(config_from_dict(copy.deepcopy(cfg_dict)), BuildEnv(torch.device("cpu"), torch.float32))
    g = torch.Generator().manual_seed(seed)
    w = {}
    for name, spec in model.tensor_specs().items():
        t = torch.randn(tuple(spec.shape), generator=g, dtype=torch.float64)
        w[name] = t * (0.3 if len(spec.shape) == 2 else 0.5)
    return w


def test_plain_prompt_equals_plain_token_by_token_and_portions():
    w = random_weights(SMALL, 3)
    ids = torch.randint(0, 61, (23,), generator=torch.Generator().manual_seed(5)).tolist()
    whole, _ = P.forward(SMALL, w, ids)
    carry, rows = None, []
    for t in ids:
        out, carry = P.forward(SMALL, w, [t], carry)
        rows.append(out)
    assert torch.allclose(torch.cat(rows), whole, rtol=1e-9, atol=1e-9)
    carry, rows, at = None, [], 0
    for c in (2, 1, 7, 2, 11):
        out, carry = P.forward(SMALL, w, ids[at:at + c], carry)
        rows.append(out)
        at += c
    assert torch.allclose(torch.cat(rows), whole, rtol=1e-9, atol=1e-9)


def test_plain_choice_stays_inside_the_kept_groups_also_with_negative_numbers():
    r = {"top": 2, "scale": 2.0, "groups": {"count": 3, "keep": 1}}
    logits = torch.tensor([0.0, 0.1, 3.0, 0.2, 0.0, 0.1], dtype=torch.float64)
    s = torch.softmax(logits, 0)
    # corrections push every number below zero; group 2 (outputs 4, 5) has the largest one
    corr = torch.tensor([-5.0, -5.0, -9.0, -9.0, -1.0, -1.2], dtype=torch.float64)
    got = P.route(logits, corr, r)
    assert [e for e, _ in got] == [5, 4] or [e for e, _ in got] == [4, 5]
    assert all(abs(wt - 2.0 * float(s[e])) < 1e-12 for e, wt in got)
    # without the limit to one group the largest corrected numbers win wherever they lie
    got = P.route(logits, corr, {"top": 2, "scale": 1.0, "groups": {"count": 3, "keep": 3}})
    assert sorted(e for e, _ in got) == [4, 5]
    got = P.route(logits, torch.zeros(6, dtype=torch.float64), {"top": 2, "scale": 1.0, "groups": {"count": 3, "keep": 2}})
    assert sorted(e for e, _ in got) == [2, 3]        # group 1 holds the best; the second output comes from it too
