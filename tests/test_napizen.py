"""Napizen without a GPU: its configuration, the tensors it asks a checkpoint for, what it keeps between steps, and the
plain implementation's mechanisms against properties that follow from their definitions."""

import copy
import math

import pytest
import torch

from tests import napizen_configs as configs
from tests.plain import napizen as plain


def test_configuration_reads_back_and_names_its_tensors(tmp_path):
    from llm_runtime_study_amd.config import config_from_dict, load_config, spec_for
    from llm_runtime_study_amd.config.napizen import NapizenConfig
    from llm_runtime_study_amd.models import DecoderModel
    from llm_runtime_study_amd.parts import PagedKVNeed

    for raw in (configs.MIXED, configs.PLAIN, configs.CORES, configs.WIDE):
        config = config_from_dict(raw)
        assert isinstance(config, NapizenConfig) and config.to_json_dict() == raw
        model = DecoderModel(spec_for(config))
        names = model.tensors()
        assert {"embed", "head", "final.norm", "l0.norm1"} <= set(names) and not any(name.endswith(".weight") for name in names)
        for index, layer in enumerate(raw["layers"]):
            m, p = layer["mixer"], f"l{index}."
            assert names[p + "mix.q"].shape == (m["heads"] * (m["dim"] + m["rot_dim"]), raw["width"])
            assert names[p + "mix.dkv"].shape == (m["kv_rank"] + m["rot_dim"], raw["width"]) and names[p + "mix.dkv.norm"].shape == (m["kv_rank"],)
            assert names[p + "mix.uk"].shape == (m["heads"] * m["dim"], m["kv_rank"]) and names[p + "mix.uv"].shape == (m["heads"] * m["vdim"], m["kv_rank"])
            assert names[p + "mix.sink"].shape == (m["heads"],) and names[p + "mix.g"].shape == (m["heads"], raw["width"])
            assert names[p + "mix.o"].shape == (raw["width"], m["heads"] * m["vdim"])
            mlp = layer["mlp"]
            if mlp is None:      # no second update; the second norm's weight is taken if a checkpoint has it all the same
                assert names[p + "norm2"].optional and not any(name.startswith(p + "mlp.") for name in names)
            elif mlp["kind"] == "dense":
                assert names[p + "mlp.gate"].shape == names[p + "mlp.up"].shape == (mlp["ff"], raw["width"]) and names[p + "mlp.down"].shape == (raw["width"], mlp["ff"])
            else:
                last = mlp["router"]["experts"] - 1
                assert names[f"{p}mlp.e{last}.gate"].shape == (mlp["expert"]["ff"], raw["width"]) and names[f"{p}mlp.e0.down"].shape == (raw["width"], mlp["expert"]["ff"])
                assert names[p + "mlp.router"].shape == (last + 1, raw["width"]) and names[p + "mlp.correction"].shape == (last + 1,)
        for layer, need in zip(raw["layers"], model.cache_needs()):
            # one row a position: the latent values and the shared rotated key part, and no value pages (an unbound model)
            assert need == PagedKVNeed(1, layer["mixer"]["kv_rank"] + layer["mixer"]["rot_dim"], None, value_dim=0)
        assert model.graph_safe() and model.plan_safe()
    folder = configs.write_folder(configs.MIXED, 3, tmp_path / "m")
    assert load_config(folder).to_json_dict() == configs.MIXED
    from tests.plain import napizen as plain_model

    stored = plain_model.load_model_dir(folder)[1]
    assert "l2.norm1" in stored and "l2.norm2" not in stored and "l1.norm2" in stored       # folders of random weights leave it out


def test_what_the_file_leaves_out_does_not_exist():
    from llm_runtime_study_amd.config import config_from_dict, spec_for

    raw = copy.deepcopy(configs.PLAIN)
    del raw["postln_alpha"], raw["embedding"]
    del raw["layers"][0]["mixer"]["scale"], raw["layers"][1]["mlp"]["router"]["scale"]
    config = config_from_dict(raw)
    spec = spec_for(config)
    assert config.alpha == 1.0 and spec.embedding_multiplier == 1.0 and spec.after_head is None
    assert config.layers[0].scale is None and config.layers[1].mlp.weight_scale == 1.0 and config.layers[1].mlp.groups == 0
    assert spec.layers[1].params["mixer"].params["position"].params["scaling"] == {"factor": 2.0, "original": 32.0, "fast": 4.0, "slow": 1.0}
    assert spec.layers[0].params["mixer"].params["position"].params["scaling"] is None
    assert spec_for(config_from_dict(configs.MIXED)).after_head.params == {"cap": 9.0}


@pytest.mark.parametrize("broken,message", [
    (lambda raw: raw["layers"][0].update(type="attention"), "unknown type"),
    (lambda raw: raw["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda raw: raw["layers"][0]["mixer"].update(rot_dim=7), "rot_dim must be even"),
    (lambda raw: raw["layers"][0]["mixer"]["rot"].update(dims=4), "rot.dims must equal rot_dim"),
    (lambda raw: raw["layers"][0]["mixer"].pop("rot"), "needs `rot`"),
    (lambda raw: raw["layers"][0]["mixer"]["rot"]["scaling"].update(factor=0), "must be positive"),
    (lambda raw: raw["layers"][0]["mlp"].update(kind="glu"), "unknown feed-forward kind"),
    (lambda raw: raw["layers"][1]["mlp"]["router"].update(top=7), "exceeds"),
    (lambda raw: raw["layers"][1]["mlp"]["router"]["groups"].update(count=4), "cannot give"),
    (lambda raw: raw["layers"][3]["mlp"]["router"]["groups"].update(keep=0), "keep must be positive"),
    (lambda raw: raw.update(logit_softcap=-1.0), "logit_softcap must be positive"),
    (lambda raw: raw["norm"].update(eps=0), "norm.eps must be positive"),
    (lambda raw: raw.update(layers=[]), "non-empty list"),
])
def test_configurations_that_cannot_run_are_refused(broken, message):
    from llm_runtime_study_amd.config import config_from_dict
    from llm_runtime_study_amd.errors import ConfigError

    raw = copy.deepcopy(configs.MIXED)
    broken(raw)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(raw)


@pytest.mark.parametrize("dims,base,scaling", [(8, 10000.0, (8.0, 64, 16.0, 2.0)), (12, 2e5, (5.0, 256, 20.0, 1.0)), (64, 1e4, (40.0, 4096, 32.0, 1.0)),
                                               (16, 2e5, (6.0, 1024, 24.0, 2.0)), (2, 30.0, (3.0, 10, 2.0, 1.0)), (32, 500.0, None)])
def test_stretched_frequencies(dims, base, scaling):
    """The position part's frequencies and magnitude against the plain implementation's; where the blend begins and ends."""
    from llm_runtime_study_amd.parts import PartSpec, create

    rot = {"dims": dims, "base": base}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    part = create("position", PartSpec("rope_interleaved", {"rotary_dim": dims, "theta": base, "scaling": rot.get("scaling")}))
    rates, factor = plain.pair_rates(rot)
    torch.testing.assert_close(part._inv_freq_host.double(), torch.tensor(rates, dtype=torch.float64), rtol=1e-6, atol=0)
    assert part.magnitude == pytest.approx(factor) and (scaling is None) == (factor == 1.0)
    untouched = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if scaling is not None:
        assert rates[0] == pytest.approx(untouched[0])                        # the fastest pair is never stretched here
        assert all(u / scaling[0] - 1e-12 <= r <= u + 1e-12 for r, u in zip(rates, untouched))


def test_plain_latent_attention_properties():
    """The sink takes weight and gives nothing back; a position sees itself and what came before; the first token's output is its
    own value times what the sink leaves."""
    g = torch.Generator().manual_seed(0)
    m = {"heads": 2, "dim": 6, "rot_dim": 4, "vdim": 5, "kv_rank": 7, "scale": 0.5, "rot": {"base": 100.0, "dims": 4}}
    shapes = {"q": (20, 9), "dkv": (11, 9), "dkv.norm": (7,), "uk": (12, 7), "uv": (10, 7), "sink": (2,), "g": (2, 9), "o": (9, 10)}
    w = {name: 0.4 * torch.randn(*shape, generator=g, dtype=torch.float64) for name, shape in shapes.items()}
    x = torch.randn(12, 9, generator=g, dtype=torch.float64)
    kept = []
    full = plain.latent_attention(x, w, m, 1e-5, kept)
    for h, i, share in kept:
        assert share.numel() == i + 1 and 0 < float(share.sum()) < 1
    assert torch.allclose(plain.latent_attention(x[:5], w, m, 1e-5), full[:5])          # causal
    low = dict(w, sink=torch.full((2,), -60.0, dtype=torch.float64))
    kept = []
    plain.latent_attention(x, low, m, 1e-5, kept)
    assert all(abs(float(share.sum()) - 1.0) < 1e-12 for _, _, share in kept)           # a sink far below every score counts for nothing
    high = dict(w, sink=torch.full((2,), 60.0, dtype=torch.float64))
    assert plain.latent_attention(x, high, m, 1e-5).abs().max() < 1e-12                 # ... and one far above takes everything


def test_plain_routing_properties():
    g = torch.Generator().manual_seed(1)
    logits, correction = torch.randn(40, 12, generator=g, dtype=torch.float64), torch.randn(12, generator=g, dtype=torch.float64) - 2.0
    router = {"experts": 12, "top": 3, "scale": 2.5, "groups": {"count": 4, "keep": 2}}
    chosen, shares = plain.choose_experts(logits, correction, router)
    for picked, share in zip(chosen, shares):
        assert len(set(picked)) == 3 and len({e // 3 for e in picked}) <= 2 and sum(share) == pytest.approx(2.5)
    free, _ = plain.choose_experts(logits, correction, {"experts": 12, "top": 3, "scale": 2.5})
    assert any(sorted(a) != sorted(b) for a, b in zip(chosen, free))                    # the groups matter for some token
    # the correction decides who is chosen and not what they weigh
    moved, moved_shares = plain.choose_experts(logits, correction + 0.75, router)
    assert moved == chosen and all(a == pytest.approx(b) for a, b in zip(shares, moved_shares))
