"""CPU tests of the Fomunex decoder: its configuration, its description as parts, its weights by
name (one number, sizes that only a tensor gives, layers that use another layer's tensors), and
the plain implementation that the GPU tests compare the engine with."""

import copy
import json

import pytest
import torch

import plain_fomunex as pf
from fomunex_configs import FOMU, make_model_dir, make_weights, random_tokens, rounding_figure, row_errors, tensor_shapes

F32_ROW = 2e-4  # the GPU tests' float32 bound on a row, relative to the logits' spread


def bf16_round(t):
    return t.bfloat16().to(t.dtype)


def _spec(cfg):
    from rapid_llm_amd.config.registry import config_from_dict

    entry, typed = config_from_dict(cfg)
    return entry, typed, entry.build_spec(typed)


@pytest.mark.parametrize("which", sorted(FOMU))
def test_configuration_round_trip_and_run_order(which):
    cfg, _page, _seed = FOMU[which]
    entry, typed, spec = _spec(cfg)
    assert entry.name == "Fomunex"
    again = type(typed).from_dict(json.loads(json.dumps(typed.to_dict())))
    assert again == typed
    owners = [i for i, layer in enumerate(cfg["layers"]) if layer.get("weights_of") is None]
    assert len(spec.layers) == len(owners)
    want = [owners.index(layer.get("weights_of", i) if layer.get("weights_of") is not None else i)
            for i, layer in enumerate(cfg["layers"])]
    assert list(spec.order()) == want
    assert spec.max_position == cfg["max_positions"]


def test_a_layer_may_name_a_layer_that_names_another():
    cfg, _page, _seed = FOMU["A"]
    chained = copy.deepcopy(cfg)
    chained["layers"].append(dict(copy.deepcopy(cfg["layers"][3]), weights_of=3))  # 6 -> 3 -> 0
    chained["layers"].insert(0, dict(copy.deepcopy(cfg["layers"][2]), weights_of=3))  # the owner comes later
    for layer in chained["layers"][1:]:
        if layer.get("weights_of") is not None:
            layer["weights_of"] += 1
    _entry, typed, spec = _spec(chained)
    assert typed.run_order() == (3, 1, 2, 3, 1, 2, 6, 1)
    assert len(spec.layers) == 4 and list(spec.order()) == [2, 0, 1, 2, 0, 1, 3, 0]
    assert spec.layers[2].checkpoint_prefix == "l3."


def test_configuration_refuses_what_the_design_does_not_have():
    from rapid_llm_amd.config.model_config import ConfigError

    cfg, _page, _seed = FOMU["A"]
    for change in (
        lambda c: c["layers"][0].update(type="convolution"),
        lambda c: c["layers"][3].update(weights_of=3),
        lambda c: (c["layers"][0].update(weights_of=3)),  # two layers that name each other
        lambda c: c["layers"][3]["mixer"].update(heads=8),  # differs from the layer whose tensors it uses
        lambda c: c["layers"][2]["mixer"].update(groups=3),
        lambda c: c["layers"][2]["mixer"].update(norm_groups=7),
        lambda c: c["layers"][1]["mlp"]["router"].update(top=7),
        lambda c: c["layers"][1]["mlp"]["expert"].pop("limit"),
        lambda c: c["layers"][0]["mixer"].update(kv_heads=3),
        lambda c: c.pop("max_positions"),
        lambda c: c["norm"].update(eps=0.0),
    ):
        broken = copy.deepcopy(cfg)
        change(broken)
        with pytest.raises(ConfigError):
            _spec(broken)


@pytest.mark.parametrize("which", sorted(FOMU))
def test_parameters_cover_the_checkpoint_tensor_by_tensor(which, tmp_path):
    """The package's own list of parameters names exactly the tensors written out in the test
    configurations, with their shapes, and nothing for a layer that uses another's."""
    from rapid_llm_amd.models.causal_lm import CausalLM
    from rapid_llm_amd.weights.loader import load_model_dir

    cfg, _page, _seed = FOMU[which]
    model = CausalLM(_spec(cfg)[2])
    named = {}
    for spec in model.param_specs():
        for src in spec.sources:
            if src.name:
                named[src.name] = spec.source_shape(src.rows)
    assert named == tensor_shapes(cfg)
    params = load_model_dir(make_model_dir(tmp_path, which), model.param_specs(), engine_dtype=torch.bfloat16,
                            device="cpu")
    assert params["final_norm.weight"].shape == () and params["final_norm.weight"].dtype == torch.float32
    for name, t in params.items():
        if name.endswith((".decay_in", ".decay_out", ".mu", ".bonus", ".conv", ".sink", ".act", ".router")):
            assert t.dtype == torch.float32, name  # what enters a recurrence, a softmax or a choice


def test_a_size_that_only_a_tensor_gives(tmp_path):
    """The inner size of the decay's two matrices is no configuration key: it is read from the
    checkpoint's tensors; a random model cannot be drawn without it."""
    from rapid_llm_amd.models.causal_lm import CausalLM
    from rapid_llm_amd.weights.loader import WeightsError, load_model_dir
    from rapid_llm_amd.weights.random_init import write_random_model

    cfg, _page, _seed = FOMU["A"]
    folder = make_model_dir(tmp_path, "A")
    bare = copy.deepcopy(cfg)
    for layer in bare["layers"]:
        layer["mixer"].pop("rank", None)
    model = CausalLM(_spec(bare)[2])
    params = load_model_dir(folder, model.param_specs(), engine_dtype=torch.float32, device="cpu")
    assert params["layers.1.mixer.decay_in"].shape == (8, 96) and params["layers.1.mixer.decay_out"].shape == (48, 8)
    with pytest.raises(ValueError):
        write_random_model(bare, 1, tmp_path / "bare")
    # given, it is checked
    other = copy.deepcopy(cfg)
    other["layers"][1]["mixer"]["rank"] = other["layers"][4]["mixer"]["rank"] = 5
    with pytest.raises(WeightsError):
        load_model_dir(folder, CausalLM(_spec(other)[2]).param_specs(), engine_dtype=torch.float32, device="cpu")
    written = write_random_model(cfg, 3, tmp_path / "drawn")
    assert set(tensor_shapes(cfg)) == set(__import__("safetensors.torch", fromlist=["load_file"]).load_file(
        str(written / "model.safetensors")))


def test_cache_needs_one_state_for_every_place():
    from rapid_llm_amd.models.causal_lm import CausalLM

    cfg, _page, _seed = FOMU["A"]
    needs = CausalLM(_spec(cfg)[2]).cache_needs()
    assert [n.kind for n in needs] == ["paged", "state", "state", "paged", "state", "state"]
    assert needs[0].window == needs[3].window == 19 and needs[3].share_with is None
    assert {s.name: s.shape for s in needs[1].states} == {"shift": (96,), "S": (3, 16, 16)}
    assert {s.name: s.shape for s in needs[2].states} == {"conv": (2, 64 + 2 * 2 * 24), "S": (4, 16, 24)}
    assert all(s.dtype == "float32" for n in needs for s in n.states)


def test_plain_tells_the_faults_the_comparison_is_there_for():
    """With the tests' weights a window one key too long or too short, scores that are not capped,
    a distance term with another slope or on the key's position alone, a sink that is left out or
    capped, a norm's weight on queries, a bonus for every token, a state that forgets the token
    before, a convolution that looks ahead, a gate behind the norm, an expert's weight on its
    output, scores that are renormalised and logits without their scale move some row by at least
    fifty times what the float32 comparison allows."""
    cfg, _page, seed = FOMU["A"]
    w = make_weights(cfg, seed, sharp=3.0)
    toks = random_tokens(90, cfg["vocab"], 9)
    want = pf.forward(cfg, w, toks)
    assert rounding_figure(pf.forward(cfg, w, toks, cast=bf16_round), want) < 0.15

    def shows(other):
        return float(row_errors(other, want).max()) > 50 * F32_ROW

    for delta in (-1, 1):
        c = copy.deepcopy(cfg)
        c["layers"][0]["mixer"]["mask"]["size"] += delta
        c["layers"][3]["mixer"]["mask"]["size"] += delta
        assert shows(pf.forward(c, w, toks)), delta
    for change in (
        lambda c: c["layers"][0]["mixer"].update(softcap=None),
        lambda c: c["layers"][1]["mlp"]["router"].update(top=1),
        lambda c: c["layers"][1]["mlp"]["expert"].update(limit=0.5),
        lambda c: c["layers"][2]["mixer"].update(norm_groups=1),
        lambda c: c.update(logit_scale=1.0),
        lambda c: c.update(logit_softcap=None),
        lambda c: c["layers"][3].pop("weights_of"),
    ):
        c = copy.deepcopy(cfg)
        change(c)
        w2 = dict(w)
        if "weights_of" not in c["layers"][3]:  # a layer of its own with other tensors
            w2.update({k.replace("l0.", "l3."): (torch.roll(v, 1, 0) if v.dim() else v) for k, v in w.items() if k.startswith("l0.")})
        assert shows(pf.forward(c, w2, toks))
    for name in ("l0.mix.sink", "l1.mix.u", "l1.mix.mu.k", "l1.mix.w0", "l2.mix.D", "l2.mix.dt_bias", "l5.mix.conv.b",
                 "pos", "l0.mlp.act"):
        w2 = dict(w)
        w2[name] = torch.zeros_like(w[name])
        assert shows(pf.forward(cfg, w2, toks)), name


def test_plain_mechanisms_one_by_one():
    """Each mechanism of the plain implementation on inputs whose answer is known."""
    eps = 1e-6
    # a window of 3: a query whose key from 3 positions back holds all the mass without the window
    # does not see it; a huge sink takes all the mass
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "scale": 20.0, "mask": {"size": 3}}
    eye = torch.eye(2, dtype=torch.float64)
    w = {"q": 40 * eye, "k": 40 * eye, "v": eye, "o": eye, "sink": torch.tensor([-50.0], dtype=torch.float64)}
    h = torch.tensor([[2.0, 0.0], [0.0, 1.0], [0.0, 1.0], [0.0, 1.0], [1.0, 0.0]], dtype=torch.float64)
    out = pf.attention(m, w, "", h, eps)
    assert out[4, 0] > 0.99 and out[4, 1] < 0.01  # only its own key matches inside the window
    m2 = dict(m, mask={"size": 5})
    out = pf.attention(m2, w, "", h, eps)
    # position 0 is seen too, at a distance that costs 2^-8 a position: its value is [2, 0]
    share = 1.0 / (1.0 + float(torch.exp(torch.tensor(4 * 2.0**-8))))
    assert abs(float(out[4, 0]) - (2.0 * share + 1.0 * (1.0 - share))) < 1e-6
    w["sink"] = torch.tensor([500.0], dtype=torch.float64)
    assert pf.attention(m, w, "", h, eps).abs().max() < 1e-9
    # the polynomial activation of a constant vector: every normed power is 1
    z = torch.full((1, 8), 3.0, dtype=torch.float64)
    assert torch.allclose(pf.polynorm(z, torch.tensor([0.5, 0.25, 2.0, -1.0], dtype=torch.float64), 0.0),
                          torch.full((1, 8), 1.75, dtype=torch.float64))
    # an expert's clamps: the gate from above only, the up value on both sides
    one = torch.ones(1, 1, dtype=torch.float64)
    ew = {"gate": 10 * one, "up": -10 * one, "down": one}
    g = 2.0
    assert torch.allclose(pf.expert(ew, "", one, 2.0), torch.tensor([[g / (1 + torch.exp(torch.tensor(-1.702 * g))) * (-2.0 + 1.0)]], dtype=torch.float64))
