"""Volonex without a GPU: its configuration (every size and constant from the file, defaults for
what a layer leaves out, errors that name the key), the order of its runs, the tensors its parts
ask for, and the rotation's frequencies against the plain implementation."""
import copy
import json

import pytest
import torch

from tests.plain import volonex_plain as P

ROT = {"base": 10000.0, "dims": 8, "scaling": {"factor": 4.0, "original": 128, "fast": 16.0, "slow": 2.0}}
CFG = {
    "architecture": "Volonex", "vocab": 77, "width": 24, "residual_mult": 0.6, "embedding": {"scale": 2.5},
    "norm": {"eps": 1e-5}, "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        {"type": "attention", "mlp": {"ff": 40, "kind": "dense", "limit": 2.0},
         "mixer": {"dim": 16, "heads": 4, "kv_heads": 2, "vdim": 8, "scale": 0.3, "mask": {"size": 20}, "rot": ROT}},
        {"type": "attention", "mlp": None,
         "mixer": {"dim": 8, "heads": 2, "kv_heads": 1, "vdim": 24, "scale": 0.5}},
        {"type": "attention", "mlp": {"ff": 12, "kind": "dense", "limit": 0.5},
         "mixer": {"dim": 8, "heads": 3, "kv_heads": 3, "vdim": 8, "scale": 0.4, "mask": {"size": 7},
                   "rot": {"base": 300.0, "dims": 8}}},
        {"type": "attention", "mlp": {"ff": 16, "kind": "dense", "limit": 1.0},
         "mixer": {"dim": 8, "heads": 2, "kv_heads": 2, "vdim": 8, "scale": 0.4}},
    ],
}


def config(data=CFG):
    import hector_engine_amd  # noqa: F401
    from hector_engine_amd.registry import config_from_dict
    return config_from_dict(copy.deepcopy(data))


def test_every_size_and_constant_comes_from_the_file():
    c = config()
    assert (c.architecture, c.vocab, c.width, c.residual_mult, c.embedding_scale, c.norm_eps) == \
        ("Volonex", 77, 24, 0.6, 2.5, 1e-5)
    a = c.layers[0].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.chunk) == (4, 2, 16, 8, 0.3, 20)
    assert (a.rot.base, a.rot.dims, a.rot.scaling.factor, a.rot.scaling.original, a.rot.scaling.fast,
            a.rot.scaling.slow) == (10000.0, 8, 4.0, 128.0, 16.0, 2.0)
    assert c.layers[1].mlp is None and c.layers[1].mixer.chunk == 0 and c.layers[1].mixer.rot is None
    assert c.layers[2].mixer.rot.scaling is None and c.layers[2].mlp.limit == 0.5
    assert c.to_dict() == json.loads(json.dumps(c.to_dict()))
    assert config(c.to_dict()).to_dict() == c.to_dict()


def test_the_runs_follow_the_loop():
    c = config()
    assert c.runs() == [(0, False), (1, False), (2, False), (1, True), (2, False), (1, True), (2, False), (3, False)]
    assert c.runs() == P.runs(CFG)
    once = copy.deepcopy(CFG)
    del once["loop"]
    assert config(once).runs() == [(l, False) for l in range(4)] == P.runs(once)
    whole = dict(copy.deepcopy(CFG), loop={"start": 0, "stop": 4, "times": 2})
    assert config(whole).runs() == P.runs(whole)
    assert [again for _, again in config(whole).runs()] == [False] * 4 + [True] + [False] * 3


@pytest.mark.parametrize("change,key", [
    (lambda d: d.pop("vocab"), "vocab"),
    (lambda d: d["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda d: d["layers"][0]["mixer"].update(kv_heads=3), "kv_heads"),
    (lambda d: d["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims"),
    (lambda d: d["layers"][0]["mixer"]["rot"].update(dims=5), "rot.dims"),
    (lambda d: d["layers"][0]["mixer"]["mask"].update(size=0), "mask.size"),
    (lambda d: d["layers"][2].update(type="recurrent"), "type"),
    (lambda d: d["layers"][0]["mlp"].update(kind="routed"), "kind"),
    (lambda d: d["layers"][0]["mlp"].pop("limit"), "limit"),
    (lambda d: d["loop"].update(stop=5), "loop"),
    (lambda d: d["loop"].update(times=0), "loop.times"),
    (lambda d: d.update(layers=[]), "layers"),
])
def test_a_configuration_that_cannot_be_used_names_its_key(change, key):
    from hector_engine_amd.config.base import ConfigError
    data = copy.deepcopy(CFG)
    change(data)
    with pytest.raises(ConfigError, match=key.replace(".", r"\.")):
        config(data)


def test_the_parts_ask_for_the_stored_tensors():
    from hector_engine_amd.parts.base import BuildEnv
    from hector_engine_amd.registry import build_model
    model = build_model(config(), BuildEnv(torch.device("cpu"), torch.float32))
    specs = {n: tuple(s.shape) for n, s in model.tensor_specs().items()}
    want = {"embed": (77, 24), "head": (77, 24), "final.norm": (24,), "final.norm.b": (24,), "final.norm.alpha": ()}
    for l, layer in enumerate(CFG["layers"]):
        m = layer["mixer"]
        for n in ("norm1",) + (("norm2",) if layer["mlp"] else ()):
            want.update({f"l{l}.{n}": (24,), f"l{l}.{n}.b": (24,), f"l{l}.{n}.alpha": ()})
        want.update({f"l{l}.mix.q": (m["heads"] * m["dim"], 24), f"l{l}.mix.k": (m["kv_heads"] * m["dim"], 24),
                     f"l{l}.mix.v": (m["kv_heads"] * m["vdim"], 24), f"l{l}.mix.o": (24, m["heads"] * m["vdim"]),
                     f"l{l}.mix.g": (m["heads"], 24), f"l{l}.mix.sink": (m["heads"],)})
        if layer["mlp"]:
            ff = layer["mlp"]["ff"]
            want.update({f"l{l}.mlp.gate": (ff, 24), f"l{l}.mlp.up": (ff, 24), f"l{l}.mlp.down": (24, ff)})
    assert specs == want
    # one cache of its own for every run, the repeated layers included
    plans = model.run_plans()
    assert len(plans) == 8 and all(p.kv is not None and p.cache_from is None for p in plans)
    assert [e.add_embedding for e in model.schedule] == [False, False, False, True, False, True, False, False]


def test_a_written_folder_holds_what_the_plain_implementation_reads(tmp_path):
    from hector_engine_amd.weights import write_random_model
    folder = write_random_model(config(), 5, str(tmp_path / "m"), "bfloat16", device=torch.device("cpu"))
    cfg, w = P.read_model(folder)
    assert cfg == config().to_dict()
    logits = P.forward(cfg, w, [3, 1, 4, 1, 5, 9, 2, 6])
    assert logits.shape == (8, 77) and torch.isfinite(logits).all()
    # token by token through the plain state gives what the whole prompt gives
    st = P.State(cfg)
    rows = torch.cat([P.step(cfg, w, st, [t]) for t in [3, 1, 4, 1, 5, 9, 2, 6]])
    assert torch.allclose(rows, logits, atol=1e-12)


@pytest.mark.parametrize("rot", [ROT, {"base": 300.0, "dims": 8},
                                 {"base": 50000.0, "dims": 32, "scaling": {"factor": 16.0, "original": 512, "fast": 40.0, "slow": 0.25}}])
def test_rotation_frequencies_against_the_plain_ones(rot):
    from hector_engine_amd.parts.base import BuildEnv, PartSpec, build_part
    params = {"head_dim": 32, "rotary_dim": rot["dims"], "theta": rot["base"], "interleaved": True}
    if "scaling" in rot:
        params["scaling"] = {"kind": "yarn", **rot["scaling"]}
    part = build_part("position", PartSpec("rotary", params), "x.", BuildEnv(torch.device("cpu"), torch.float32))
    f, mult = P.rotary_frequencies(rot)
    got, dims = part.rotary()
    assert dims == rot["dims"] and torch.allclose(got.double(), f, rtol=1e-7)
    assert abs(part.mscale - mult) < 1e-12


def test_chunks_are_counted_from_position_zero():
    assert P.sees(23, 20, 20) and not P.sees(23, 19, 20) and P.sees(19, 0, 20) and not P.sees(20, 19, 20)
    assert P.sees(5, 5, 20) and not P.sees(4, 5, 20)
