"""CPU tests of the Miborax decoder: its configuration, its description as parts, its weights by
name, how long a cache that several layers read keeps its rows, and the plain implementation
that the GPU tests compare the engine with."""

import copy

import pytest
import torch

import plain_miborax as pm
from miborax_configs import (
    BF16_ROWS_BEYOND,
    MIBO,
    make_weights,
    random_tokens,
    rounding_figure,
    row_errors,
    share_beyond,
    tensor_shapes,
)

F32_ROW = 2e-4  # the GPU tests' float32 bound on a row, relative to the logits' spread


def bf16_round(t):
    return t.bfloat16().to(t.dtype)


def test_plain_tells_the_faults_the_comparison_is_there_for():
    """With the tests' weights a window one key too long or too short, a softmax without its
    extra term or with that term scaled like a score, heads that are not gated, pairs rotated
    the other way round or halves paired instead of neighbours, a rotated key part that is
    normed like the latent, a router without its bias, an expert too few, a norm without its
    bias and an unscaled embedding move some row by at least fifty times what the float32
    comparison allows, and most of them far more rows than the bfloat16 comparison allows."""
    cfg, _page, seed = MIBO["A"]
    w = make_weights(cfg, seed, sharp=3.0)
    toks = random_tokens(150, cfg["vocab"], 9)
    want = pm.forward(cfg, w, toks)
    figure = rounding_figure(pm.forward(cfg, w, toks, cast=bf16_round), want)
    assert figure < 0.04

    def shows(other, in_bfloat16=True):
        assert float(row_errors(other, want).max()) > 50 * F32_ROW
        return not in_bfloat16 or share_beyond(other, want, figure) > 2 * BF16_ROWS_BEYOND

    for layer in (0, 2, 3):
        for delta in (-1, 1):
            c = copy.deepcopy(cfg)
            c["layers"][layer]["mixer"]["mask"]["size"] += delta
            assert shows(pm.forward(c, w, toks)), (layer, delta)
    c = copy.deepcopy(cfg)
    c["layers"][0]["mlp"]["router"]["top"] -= 1
    assert shows(pm.forward(c, w, toks))
    c = copy.deepcopy(cfg)
    c["embedding"]["scale"] = 1.0
    assert shows(pm.forward(c, w, toks))
    for name in ("l1.norm1.b", "l3.norm2.b", "final.norm.b", "l0.mlp.router.b", "l1.mix.g"):
        w2 = dict(w)
        w2[name] = torch.zeros_like(w[name])
        assert shows(pm.forward(cfg, w2, toks)), name
    for i in range(len(cfg["layers"])):
        # where few keys carry a query's weight the extra term moves few rows, those by much
        w2 = dict(w)
        w2[f"l{i}.mix.sink"] = w[f"l{i}.mix.sink"] - 30.0  # as good as no extra term
        assert shows(pm.forward(cfg, w2, toks), in_bfloat16=False), i
        w2 = dict(w)
        w2[f"l{i}.mix.sink"] = (w[f"l{i}.mix.sink"].float() * cfg["layers"][i]["mixer"]["scale"]).bfloat16()
        assert shows(pm.forward(cfg, w2, toks), in_bfloat16=False), i

    def half_split(x, positions, base, dims):
        out = x.clone()
        i = torch.arange(dims // 2, dtype=torch.float64)
        angle = positions.double()[:, None] * base ** (-2.0 * i / dims)
        cos, sin = torch.cos(angle).to(x.dtype), torch.sin(angle).to(x.dtype)
        while cos.dim() < x.dim():
            cos, sin = cos.unsqueeze(1), sin.unsqueeze(1)
        u, v = x[..., : dims // 2], x[..., dims // 2:dims]
        out[..., : dims // 2] = u * cos - v * sin
        out[..., dims // 2:dims] = v * cos + u * sin
        return out

    def backwards(x, positions, base, dims):
        return saved_rotate(x, -positions, base, dims)

    def from_one(x, positions, base, dims):
        return saved_rotate(x, positions + 1, base, dims)

    def all_normed(h, m, w_, p, eps, positions, cast):
        c, kr = saved_latent(h, m, w_, p, eps, positions, cast)
        return c, kr / torch.sqrt((kr * kr).mean(-1, keepdim=True) + eps)

    saved_rotate, saved_latent = pm.rotate_pairs, pm.latent_of
    try:
        for broken in (half_split, backwards):
            pm.rotate_pairs = broken
            assert shows(pm.forward(cfg, w, toks)), broken.__name__
        # a rotation that counts positions from 1 turns queries and keys alike: scores see
        # differences of positions only, and nothing moves
        pm.rotate_pairs = from_one
        assert float(row_errors(pm.forward(cfg, w, toks), want).max()) < 1e-4
        pm.rotate_pairs = saved_rotate
        pm.latent_of = all_normed
        assert shows(pm.forward(cfg, w, toks))
    finally:
        pm.rotate_pairs, pm.latent_of = saved_rotate, saved_latent


def test_a_reader_of_another_layers_rows_is_not_a_layer_with_rows_of_its_own():
    """Layer 4 of configuration A reads layer 3's rows; with a projection of its own (drawn at
    random) its output is another."""
    cfg, _page, seed = MIBO["A"]
    w = make_weights(cfg, seed, sharp=3.0)
    toks = random_tokens(40, cfg["vocab"], 11)
    want = pm.forward(cfg, w, toks)
    c = copy.deepcopy(cfg)
    del c["layers"][4]["mixer"]["kv_from"]
    w2 = dict(w)
    w2["l4.mix.dkv"] = w["l3.mix.dkv"].flip(0)
    w2["l4.mix.dkv.norm"] = w["l3.mix.dkv.norm"]
    assert float(row_errors(pm.forward(c, w2, toks), want).median()) > 0.05


def test_plain_mask_sink_and_rotation():
    seen = pm.visible(torch.arange(12), 4)
    for i in range(12):
        for j in range(12):
            assert bool(seen[i, j]) == (0 <= i - j < 4)
    assert pm.visible(torch.arange(5), 0).equal(torch.ones(5, 5).tril().bool())
    # the extra term is a softmax over one more key whose score is the head's number and whose
    # weight is dropped
    s = torch.randn(3, 6, 9, dtype=torch.float64) * 3
    sink = torch.tensor([-2.0, 0.0, 4.0], dtype=torch.float64)
    mask = pm.visible(torch.arange(9), 3)[3:]
    masked = s.masked_fill(~mask[None], float("-inf"))
    with_key = torch.softmax(torch.cat([masked, sink[:, None, None].expand(3, 6, 1)], dim=-1), dim=-1)
    torch.testing.assert_close(pm.sink_softmax(s, mask, sink), with_key[..., :-1])
    # very negative scores: the weights vanish instead of summing to one
    gone = pm.sink_softmax(torch.full((1, 1, 3), -50.0, dtype=torch.float64), torch.ones(1, 3, dtype=torch.bool),
                           torch.zeros(1, dtype=torch.float64))
    assert float(gone.sum()) < 1e-20
    # rotation: position 0 leaves a vector as it is; lengths of pairs are kept; channels beyond
    # `dims` pass; scores of two rotated vectors depend on the difference of their positions
    x = torch.randn(4, 2, 12, dtype=torch.float64)
    torch.testing.assert_close(pm.rotate_pairs(x, torch.zeros(4, dtype=torch.long), 100.0, 8), x)
    y = pm.rotate_pairs(x, torch.tensor([3, 50, 7, 1000]), 100.0, 8)
    assert torch.equal(y[..., 8:], x[..., 8:])
    torch.testing.assert_close(y[..., 0:8:2] ** 2 + y[..., 1:8:2] ** 2, x[..., 0:8:2] ** 2 + x[..., 1:8:2] ** 2)
    a, b = torch.randn(1, 8, dtype=torch.float64), torch.randn(1, 8, dtype=torch.float64)
    s1 = (pm.rotate_pairs(a, torch.tensor([9]), 50.0, 8) * pm.rotate_pairs(b, torch.tensor([4]), 50.0, 8)).sum()
    s2 = (pm.rotate_pairs(a, torch.tensor([25]), 50.0, 8) * pm.rotate_pairs(b, torch.tensor([20]), 50.0, 8)).sum()
    torch.testing.assert_close(s1, s2, rtol=1e-5, atol=1e-5)  # the angle is a float32 product
    # pair (1, 0) at angle a becomes (cos a, sin a)
    e = torch.zeros(1, 2, dtype=torch.float64)
    e[0, 0] = 1.0
    r = pm.rotate_pairs(e, torch.tensor([1]), 7.0, 2)
    torch.testing.assert_close(r, torch.tensor([[0.5403023058681398, 0.8414709848078965]], dtype=torch.float64))


def test_plain_norms_and_activation():
    x = torch.randn(5, 33, dtype=torch.float64) * 3 + 2
    w, b = torch.randn(33, dtype=torch.float64), torch.randn(33, dtype=torch.float64)
    want = torch.nn.functional.layer_norm(x, (33,), w, b, 1e-5)
    torch.testing.assert_close(pm.layer_norm(x, w, b, 1e-5), want)
    r = pm.rms_norm(x, w, 1e-5)
    torch.testing.assert_close(r, x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w)


def test_the_mixer_over_the_latent_rows_equals_the_mixer_over_keys_and_values():
    """The form the engine computes (queries through the key matrices, softmax weights over the
    latent rows, value matrices last) against the design's own statement, for every layer of
    every configuration."""
    for which, (cfg, _page, seed) in MIBO.items():
        w = {k: v.double() for k, v in make_weights(cfg, seed, sharp=2.0).items()}
        positions = torch.arange(50)
        latents = {}
        for i, layer in enumerate(cfg["layers"]):
            m, p = layer["mixer"], f"l{i}.mix."
            h = torch.randn(50, cfg["width"], dtype=torch.float64)
            if "kv_from" in m:
                latent = latents[m["kv_from"]]
            else:
                latent = latents[i] = pm.latent_of(h, m, w, p, 1e-6, positions, pm.identity)
            a = pm.latent_attention(h, m, w, p, 1e-6, positions, latent)
            b = pm.absorbed_attention(h, m, w, p, 1e-6, positions, latent)
            torch.testing.assert_close(a, b, rtol=1e-9, atol=1e-9)


def test_plain_experts_equal_their_dense_form():
    """The weighted sum over a token's chosen experts equals two dense products over all experts'
    hidden units with the unchosen ones' weights at zero (the form the engine computes), and the
    weights are a softmax over the chosen logits alone."""
    torch.manual_seed(3)
    width, experts, ff, top = 24, 5, 7, 2
    h = torch.randn(11, width, dtype=torch.float64)
    w = {"router": torch.randn(experts, width, dtype=torch.float64), "router.b": torch.randn(experts, dtype=torch.float64) * 2}
    for e in range(experts):
        w[f"e{e}.gate"] = torch.randn(ff, width, dtype=torch.float64)
        w[f"e{e}.up"] = torch.randn(ff, width, dtype=torch.float64)
        w[f"e{e}.down"] = torch.randn(width, ff, dtype=torch.float64)
    cfg = {"router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    want = pm.experts(h, cfg, w, "")
    chosen, weight = pm.route(h, cfg, w, "")
    torch.testing.assert_close(weight.sum(dim=1), torch.ones(11, dtype=torch.float64))
    everyone = torch.softmax(h @ w["router"].T + w["router.b"], dim=-1)
    picked = everyone.gather(1, chosen)
    torch.testing.assert_close(weight, picked / picked.sum(dim=1, keepdim=True))
    without_bias = torch.topk(h @ w["router"].T, top, dim=-1).indices
    assert not torch.equal(without_bias.sort(dim=1).values, chosen.sort(dim=1).values)  # the bias decides some
    dense = torch.zeros(11, experts, dtype=torch.float64).scatter_(1, chosen, weight)
    gate = torch.cat([w[f"e{e}.gate"] for e in range(experts)])
    up = torch.cat([w[f"e{e}.up"] for e in range(experts)])
    down = torch.cat([w[f"e{e}.down"] for e in range(experts)], dim=1)
    g = h @ gate.T
    hidden = g * torch.sigmoid(g) * (h @ up.T) * dense.repeat_interleave(ff, dim=1)
    torch.testing.assert_close(hidden @ down.T, want)


def test_configuration_round_trip_and_description():
    from rapid_llm_amd.config.registry import config_from_dict

    for which, (cfg, _page, _seed) in MIBO.items():
        entry, parsed = config_from_dict(cfg)
        assert entry.name == "Miborax"
        assert config_from_dict(parsed.to_dict())[1] == parsed
        assert (parsed.width, parsed.vocab, parsed.embedding_scale, parsed.norm_eps) == (
            cfg["width"], cfg["vocab"], cfg["embedding"]["scale"], cfg["norm"]["eps"])
        spec = entry.build_spec(parsed)
        assert spec.order() == tuple(range(len(cfg["layers"])))
        for i, (layer, listed, described) in enumerate(zip(parsed.layers, cfg["layers"], spec.layers)):
            m = listed["mixer"]
            assert layer.mixer.window == (m.get("mask") or {}).get("size", 0)
            assert layer.mixer.kv_from == m.get("kv_from")
            assert described.share_cache_with == m.get("kv_from")
            p = described.mixer.params
            assert (p["num_heads"], p["head_dim"], p["rot_dim"], p["value_dim"], p["kv_rank"], p["softmax_scale"]) == (
                m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"])
            assert p["q_rank"] == m.get("q_rank", 0) and p["gate"] == (listed["type"] == "latent_attention")
            assert p["owns_latent"] == ("kv_from" not in m)
            assert described.position.params["theta"] == m["rot"]["base"]
            assert described.position.params["rotary_dim"] == m["rot"]["dims"]
            assert (described.feed_forward is None) == (listed["mlp"] is None)
            if listed["mlp"] is not None:
                f = described.feed_forward.params
                assert (f["num_experts"], f["top"], f["expert_size"]) == (
                    listed["mlp"]["router"]["experts"], listed["mlp"]["router"]["top"], listed["mlp"]["expert"]["ff"])
            # the cache keeps the longest view of the rows: the layer's own and its readers'
            owner = i if layer.mixer.kv_from is None else layer.mixer.kv_from
            views = [parsed.layers[owner].mixer.window] + [
                other.mixer.window for other in parsed.layers if other.mixer.kv_from == owner]
            assert p["cache_window"] == (0 if 0 in views else max(views))
    a = config_from_dict(MIBO["A"][0])[1]
    assert [a.cache_window(i) for i in (0, 3)] == [41, 7]
    assert config_from_dict(MIBO["C"][0])[1].cache_window(0) == 0


def test_every_checkpoint_tensor_is_claimed_once_and_shapes_agree():
    from rapid_llm_amd.config.registry import config_from_dict
    from rapid_llm_amd.models.causal_lm import model_param_specs
    from rapid_llm_amd.weights.loader import WeightsError, load_params

    for which, (cfg, _page, seed) in MIBO.items():
        entry, parsed = config_from_dict(cfg)
        spec = entry.build_spec(parsed)
        specs = model_param_specs(spec)
        named = {src.name: spec_.source_shape(src.rows) for spec_ in specs for src in spec_.sources if src.name}
        assert named.pop("head") == (cfg["vocab"], cfg["width"])  # stands for the embedding's table
        assert named == tensor_shapes(cfg)
        weights = make_weights(cfg, seed)
        params = load_params(specs, weights.items(), engine_dtype=torch.bfloat16, device="cpu")
        assert params["output.weight"] is params["embed.weight"]
        for spec_ in specs:
            assert tuple(params[spec_.name].shape) == spec_.shape
            offset = 0
            for src in spec_.sources:
                part = params[spec_.name].narrow(spec_.axis, offset, src.rows)
                if src.name and src.name != "head":
                    assert torch.equal(part.float(), weights[src.name].float())
                elif not src.name:
                    assert not part.any()  # padding of a packed matrix is zeros
                offset += src.rows
        routers = [s for s in specs if s.role == "matrix_f32"]
        assert routers and all(params[s.name].dtype == torch.float32 for s in routers)
        # a checkpoint that still carries the second norm of a layer without a feed-forward loads
        extra = dict(weights)
        for i, layer in enumerate(cfg["layers"]):
            if layer["mlp"] is None:
                extra[f"l{i}.norm2"] = torch.ones(cfg["width"])
                extra[f"l{i}.norm2.b"] = torch.zeros(cfg["width"])
        load_params(specs, extra.items(), engine_dtype=torch.bfloat16, device="cpu", ignore_rules=spec.ignore_tensors)
        broken = dict(weights)
        del broken["final.norm.b"]
        broken["l0.mix.extra"] = torch.zeros(3)
        with pytest.raises(WeightsError) as err:
            load_params(specs, broken.items(), engine_dtype=torch.bfloat16, device="cpu")
        assert any("final.norm.b" in m for m in err.value.missing) and any("l0.mix.extra" in u for u in err.value.unexpected)


def test_random_weights_for_the_design(tmp_path):
    from safetensors.torch import load_file

    from rapid_llm_amd.weights.random_init import write_random_model

    for which in ("A", "D"):
        cfg = MIBO[which][0]
        out = write_random_model(cfg, 5, tmp_path / which)
        tensors = load_file(str(out / "model.safetensors"))
        assert {k: tuple(v.shape) for k, v in tensors.items()} == tensor_shapes(cfg)


def test_configuration_refuses_what_the_design_does_not_have():
    from rapid_llm_amd.config.model_config import ConfigError
    from rapid_llm_amd.config.registry import config_from_dict

    base = MIBO["A"][0]
    for change in (
        lambda c: c["layers"][0].__setitem__("type", "convolution"),
        lambda c: c["layers"][0]["mixer"].pop("mask"),
        lambda c: c["layers"][0]["mixer"].__setitem__("q_rank", 16),
        lambda c: c["layers"][1]["mixer"].pop("q_rank"),
        lambda c: c["layers"][1]["mixer"].__setitem__("kv_from", 0),
        lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 2),
        lambda c: c["layers"][2]["mixer"].__setitem__("kv_from", 3),
        lambda c: c["layers"][4]["mixer"].__setitem__("kv_from", 2),  # a reader itself
        lambda c: c["layers"][2]["mixer"].__setitem__("kv_rank", 48),  # other rows than layer 0 caches
        lambda c: c["layers"][2]["mixer"]["rot"].__setitem__("base", 3.0),
        lambda c: c["layers"][0]["mixer"].__setitem__("rot_dim", 7),
        lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 64),
        lambda c: c["layers"][0]["mixer"].__setitem__("heads", 0),
        lambda c: c["layers"][0]["mlp"].__setitem__("kind", "dense"),
        lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 7),
        lambda c: c["layers"][0]["mlp"].pop("expert"),
        lambda c: c["norm"].pop("eps"),
        lambda c: c.__setitem__("layers", []),
    ):
        cfg = copy.deepcopy(base)
        change(cfg)
        with pytest.raises(ConfigError):
            config_from_dict(cfg)


def test_layers_that_share_rows_share_a_cache_group_with_the_longest_view():
    """What the cache manager is told: a reader has no pages of its own, and the rows it reads
    are kept for as long as the longest view on them needs."""
    from rapid_llm_amd.config.registry import config_from_dict
    from rapid_llm_amd.parts import MIXERS, POSITION_ENCODINGS

    entry, parsed = config_from_dict(MIBO["A"][0])
    spec = entry.build_spec(parsed)
    needs = []
    for layer in spec.layers:
        position = POSITION_ENCODINGS.create(layer.position.kind, **layer.position.params)
        mixer = MIXERS.create(layer.mixer.kind, position=position, **layer.mixer.params)
        needs.append(mixer.cache_need())
    assert [n.window for n in needs] == [41, 0, 41, 7, 7]
    # one shared row a token: the latent with the rotated part as keys, the latent transposed as values
    assert needs[0].paged[0].shape == (1, 64) and needs[0].paged[1].shape == (1, 32)
    assert needs[1].paged[0].shape == (1, 96) and needs[1].paged[1].shape == (1, 80)
