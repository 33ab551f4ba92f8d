"""Fosulix without a GPU: the configuration reader and its errors, the list of tensors, which layers share a cache,
the stretched rotary frequencies, and the plain implementation's own consistency."""
import copy
import math

import pytest
import torch

from leone_amd.architectures import config_from_dict, model_spec_for
from leone_amd.config import ConfigError
from leone_amd.config.fosulix import FosulixConfig, LatentAttentionConfig
from leone_amd.parts import DecoderModel
from leone_amd.parts.latent import LatentNeed
from tests import fosulix_util as fu
from tests.plain import fosulix_plain as plain


@pytest.mark.parametrize("name", list(fu.SMALL))
def test_configuration_reads_back_and_names_the_design_tensors(name):
    raw = fu.SMALL[name]
    config = config_from_dict(raw)
    assert isinstance(config, FosulixConfig) and config.architecture == "Fosulix"
    assert config_from_dict(config.to_dict()) == config
    assert config.vocab_size == raw["vocab"] and config.max_position_embeddings == raw["max_positions"]
    model = DecoderModel(model_spec_for(config), torch.float32, "cpu")
    assert {s.name: tuple(s.shape) for s in model.tensor_specs()} == fu.tensor_shapes(raw)
    assert model.graph_safe
    assert model.spec.head is None and model.spec.embedding_scale == raw["embedding"]["scale"]


def test_a_reader_of_latents_shares_the_owner_s_pages_and_keeps_its_own_convolution():
    raw = fu.SMALL["A"]
    config = config_from_dict(raw)
    model = DecoderModel(model_spec_for(config), torch.float32, "cpu")
    needs = model.cache_needs()
    # layers 2 and 4 read the latents of layers 0 and 3: no pages of their own, but inputs of their own convolution
    assert (2, "mixer") not in needs and (4, "mixer") not in needs
    assert all((i, "conv1") in needs for i in range(5))
    assert needs[(0, "conv1")].shape == (raw["canon"]["taps"] - 1, raw["width"])
    # the owner's cache keeps the widest window of its readers; a layer without a mask keeps everything
    assert needs[(0, "mixer")] == LatentNeed(24, 8, 33) and needs[(3, "mixer")] == LatentNeed(40, 4, None)
    assert config.latent_retention(0) == 33 and config.latent_retention(3) is None
    assert needs[(1, "mixer")].shape == (3, 12 * 20)
    runs = model.schedule
    assert runs[2].borrow == {"mixer": 0} and runs[4].borrow == {"mixer": 3} and runs[0].borrow is None
    assert all(run.cache == i and run.writes for i, run in enumerate(runs))
    assert model.layers[2].mixer.shared_kv and model.layers[2].mixer.window == 33 and model.layers[0].mixer.window == 20


def test_defaults_where_the_configuration_is_silent():
    raw = copy.deepcopy(fu.SMALL["B"])
    del raw["max_positions"]
    config = config_from_dict(raw)
    assert config.max_positions == 32768
    attention = config.layers[4].mixer
    assert isinstance(attention, LatentAttentionConfig) and attention.window is None and attention.kv_from is None
    assert config.layers[1].mixer.rot_dims == 8 and config.layers[1].mixer.rot_dim == 16
    assert config.layers[0].mlp.group_count == 9 and config.layers[4].mlp.group_count == 1
    assert config.layers[2].mlp is None
    assert config_from_dict(fu.SMALL["A"]).layers[3].mixer.rot_scaling is None


BROKEN = [
    (lambda r: r.pop("residual_mult"), "residual_mult"),
    (lambda r: r["embedding"].pop("scale"), "embedding.scale"),
    (lambda r: r["canon"].update(taps=1), "canon.taps"),
    (lambda r: r["layers"][0].update(type="attention"), "layers[0].type"),
    (lambda r: r["layers"][0]["mixer"].pop("kv_rank"), "layers[0].mixer.kv_rank"),
    (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=7), "layers[0].mixer.rot.dims"),
    (lambda r: r["layers"][0]["mixer"]["rot"]["scaling"].pop("fast"), "layers[0].mixer.rot.scaling.fast"),
    (lambda r: r["layers"][0]["mixer"]["mask"].update(size=0), "layers[0].mixer.mask.size"),
    (lambda r: r["layers"][2]["mixer"].update(kv_from=2), "layers[2].mixer.kv_from"),
    (lambda r: r["layers"][2]["mixer"].update(kv_from=1), "layers[2].mixer.kv_from"),
    (lambda r: r["layers"][2]["mixer"].update(kv_rank=30), "layers[2].mixer.kv_from"),
    (lambda r: r["layers"][4]["mixer"].update(kv_from=2), "layers[4].mixer.kv_from"),
    (lambda r: r["layers"][1]["mixer"].pop("vdim"), "layers[1].mixer.vdim"),
    (lambda r: r["layers"][0]["mlp"].update(kind="dense"), "layers[0].mlp.kind"),
    (lambda r: r["layers"][0]["mlp"]["expert"].pop("limit"), "layers[0].mlp.expert.limit"),
    (lambda r: r["layers"][0]["mlp"]["router"].update(top=7), "layers[0].mlp.router.top"),
    (lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(count=4), "layers[0].mlp.router.groups"),
    (lambda r: r["layers"][0]["mlp"]["router"]["groups"].update(keep=1, count=6), "layers[0].mlp.router.groups"),
    (lambda r: r["layers"][0]["mlp"]["router"].pop("scale"), "layers[0].mlp.router.scale"),
]


@pytest.mark.parametrize("change,field", BROKEN, ids=[f"{n}:{field}" for n, (_, field) in enumerate(BROKEN)])
def test_errors_name_the_key(change, field):
    raw = copy.deepcopy(fu.SMALL["A"])
    change(raw)
    with pytest.raises(ConfigError) as error:
        config_from_dict(raw)
    assert error.value.field == field, str(error.value)


def test_stretched_frequencies_against_the_plain_ones():
    from leone_amd.parts import POSITIONS, PartSpec
    cases = [(32, 50000.0, 4.0, 2048, 16.0, 2.0), (8, 77.0, 4.0, 32, 8.0, 2.0), (64, 1e6, 40.0, 4096, 1.0, 1.0),
             (4, 10.0, 2.0, 16, 4.0, 1.0), (16, 500.0, 1.0, 64, 32.0, 1.0)]
    for dims, base, factor, original, fast, slow in cases:
        scaling = {"factor": factor, "original": original, "fast": fast, "slow": slow}
        part = POSITIONS.build(PartSpec("rope_scaled_adjacent", {"rotary_dim": dims, "theta": base, **scaling}))
        part.prepare(300, "cpu")
        freq, grow = plain.rotary_frequencies(dims, base, scaling)
        assert grow == pytest.approx(0.1 * math.log(factor) + 1.0)
        angle = torch.arange(300, dtype=torch.float64)[:, None] * torch.tensor(freq, dtype=torch.float64)[None, :]
        cos, sin = part.tables()
        assert cos.shape == (300, dims // 2)
        assert torch.allclose(cos.double(), torch.cos(angle) * grow, atol=1e-6)
        assert torch.allclose(sin.double(), torch.sin(angle) * grow, atol=1e-6)
    # the first pairs keep their frequency, the last are slowed by the whole factor
    freq, _ = plain.rotary_frequencies(32, 50000.0, {"factor": 4.0, "original": 2048, "fast": 16.0, "slow": 1.0})
    assert freq[0] == 1.0 and freq[-1] == pytest.approx(50000.0 ** (-30 / 32) / 4.0)


def test_plain_pieces_agree_with_one_another():
    """The plain model walked whole and its prefix agree (causality), a reader with the owner's window sees what the
    owner sees, and the router never leaves the open groups."""
    raw = fu.SMALL["C"]
    weights = {k: v.float() for k, v in fu.make_weights(raw, 3, torch.float32).items()}
    tokens = list(range(3, 60))
    whole = plain.forward(raw, weights, tokens)
    assert torch.allclose(plain.forward(raw, weights, tokens[:31]), whole[:31], atol=1e-9)
    r = {"experts": 12, "top": 3, "scale": 2.0, "groups": {"count": 4, "keep": 2}}
    gen = torch.Generator().manual_seed(0)
    h, router = torch.randn(40, 16, generator=gen, dtype=torch.float64), torch.randn(12, 16, generator=gen, dtype=torch.float64)
    chosen, weight = plain.route(h, router, r)
    s = torch.sigmoid(h @ router.T)
    for row in range(40):
        groups = {e // 3 for e in chosen[row].tolist()}
        assert len(groups) <= 2
        score = sorted(((s[row, g * 3:g * 3 + 3].topk(2).values.sum().item(), g) for g in range(4)), reverse=True)
        assert groups <= {g for _, g in score[:2]}
        assert torch.allclose(weight[row], s[row, chosen[row]] * 2.0)
