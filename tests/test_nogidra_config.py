"""Nogidra without a GPU: the configuration reader and its errors, the list of tensors, what every layer keeps between
steps, the reordering that serves half-split pairs to kernels that turn neighbours, and the plain implementation's own
consistency."""
import copy
import math

import pytest
import torch

from leone_amd.architectures import config_from_dict, model_spec_for
from leone_amd.architectures.nogidra import distance_slopes
from leone_amd.config import ConfigError
from leone_amd.config.nogidra import BiasedAttentionConfig, DenseConfig, MixtureConfig, NogidraConfig, ParallelConfig
from leone_amd.parts import DecoderModel
from leone_amd.parts.base import KvNeed, StateNeed
from leone_amd.parts.latent import LatentNeed
from tests import nogidra_util as nu
from tests.plain import nogidra_plain as plain


@pytest.mark.parametrize("name", list(nu.SMALL))
def test_configuration_reads_back_and_names_the_design_tensors(name):
    raw = nu.SMALL[name]
    config = config_from_dict(raw)
    assert isinstance(config, NogidraConfig) and config.architecture == "Nogidra"
    assert config_from_dict(config.to_dict()) == config and config.to_dict() == raw
    assert config.vocab_size == raw["vocab"] and config.max_position_embeddings == raw["max_positions"]
    model = DecoderModel(model_spec_for(config), torch.float32, "cpu")
    assert {s.name: tuple(s.shape) for s in model.tensor_specs()} == nu.tensor_shapes(raw)
    assert model.graph_safe
    assert model.spec.head == "head" and model.spec.logit_cap == raw.get("logit_softcap")


def test_what_every_layer_keeps_between_steps():
    raw = nu.SMALL["A"]
    model = DecoderModel(model_spec_for(config_from_dict(raw)), torch.float32, "cpu")
    needs = model.cache_needs()
    # attention behind convolutions: paged keys and values, and the last taps - 1 projected rows of q, k and v
    assert needs[(0, "kv")] == KvNeed(2, 16, 20, value_dim=24) and needs[(0, "conv")] == StateNeed((2, 4 * 16 + 2 * 16 + 2 * 24))
    # side by side: the left branch's keys; the right branch's convolution inputs (x, B and C) and its memory
    assert needs[(1, "left")] == KvNeed(2, 16, 33)
    assert needs[(1, "right", "conv")] == StateNeed((1, 3 * 8 + 2 * 3 * 12)) and needs[(1, "right", "memory")] == StateNeed((3, 12 * 8))
    assert needs[2] == LatentNeed(24, 8, 7)
    assert needs[3] == KvNeed(1, 8, None)                       # no convolution, no window: a plain key/value cache
    assert needs[(4, "left")] == KvNeed(1, 24, None, value_dim=8) and needs[(4, "right", "memory")] == StateNeed((4, 20 * 12))
    first = model.layers[0].mixer
    assert first.slope_values == [2.0 ** -2, 2.0 ** -4, 2.0 ** -6, 2.0 ** -8] and first.query_factor == (0.7, 8)
    assert model.layers[3].mixer.query_factor is None and model.layers[3].mixer.conv is None
    assert model.layers[2].feed_forward is None and model.layers[2].norm2 is None
    side = model.layers[1].mixer
    assert side.weights == {"left": 0.8, "right": -0.6} and side.branches["left"].wide_norm and side.branches["left"].bias_names
    assert distance_slopes(1) == [2.0 ** -8] and distance_slopes(3)[1] == pytest.approx(2.0 ** (-16 / 3))


def test_defaults_where_the_configuration_is_silent():
    raw = copy.deepcopy(nu.SMALL["B"])
    del raw["max_positions"]
    config = config_from_dict(raw)
    assert config.max_positions == 32768 and config.logit_softcap is None
    assert isinstance(config.layers[0].mixer, ParallelConfig) and config.layers[0].mixer.right.norm_groups == 2
    assert config.layers[3].mixer.window is None and config.layers[2].mlp is None
    assert isinstance(config.layers[0].mlp, DenseConfig) and isinstance(config.layers[1].mlp, MixtureConfig)
    plain_attention = config_from_dict(nu.SMALL["A"]).layers[3].mixer
    assert isinstance(plain_attention, BiasedAttentionConfig)
    assert plain_attention.taps is None and plain_attention.temp_every is None and plain_attention.window is None
    bare = copy.deepcopy(nu.SMALL["A"])
    for key in ("kv_heads", "vdim", "scale"):
        del bare["layers"][0]["mixer"][key]
    first = config_from_dict(bare).layers[0].mixer
    assert (first.kv_heads, first.vdim, first.scale) == (4, 16, 0.25)       # as many as heads, the keys' size, 16 ** -0.5
    # a file may hold the second norm of a layer without a feed-forward; nothing else goes unused
    assert model_spec_for(config_from_dict(nu.SMALL["A"])).ignore_tensors == ("l2.norm2",)


BROKEN = [
    (lambda r: r.pop("width"), "width"),
    (lambda r: r["norm"].pop("eps"), "eps"),
    (lambda r: r.update(logit_softcap=-1.0), "logit_softcap"),
    (lambda r: r["layers"][0].update(type="hgrn2"), "layers[0].type"),
    (lambda r: r["layers"][0]["mixer"].pop("dim"), "layers[0].mixer.dim"),
    (lambda r: r["layers"][0]["mixer"].update(vdim=0), "layers[0].mixer.vdim"),
    (lambda r: r["layers"][0]["mixer"].update(kv_heads=3), "layers[0].mixer.kv_heads"),
    (lambda r: r["layers"][0]["mixer"].update(conv=1), "layers[0].mixer.conv"),
    (lambda r: r["layers"][0]["mixer"]["q_temp"].update(every=0), "layers[0].mixer.q_temp.every"),
    (lambda r: r["layers"][0]["mixer"]["q_temp"].pop("coef"), "layers[0].mixer.q_temp.coef"),
    (lambda r: r["layers"][0]["mixer"]["mask"].update(size=0), "layers[0].mixer.mask.size"),
    (lambda r: r["layers"][0]["mlp"].pop("ff"), "layers[0].mlp.ff"),
    (lambda r: r["layers"][0]["mlp"].update(kind="glu"), "layers[0].mlp.kind"),
    (lambda r: r["layers"][1]["mixer"].pop("left_scale"), "layers[1].mixer.left_scale"),
    (lambda r: r["layers"][1]["mixer"]["left"]["rot"].update(dims=18), "layers[1].mixer.left.rot.dims"),
    (lambda r: r["layers"][1]["mixer"]["left"]["rot"].update(base=1.0), "layers[1].mixer.left.rot.base"),
    (lambda r: r["layers"][1]["mixer"]["right"].update(groups=2), "layers[1].mixer.right.groups"),
    (lambda r: r["layers"][1]["mixer"]["right"].update(norm_groups=5), "layers[1].mixer.right.norm_groups"),
    (lambda r: r["layers"][1]["mixer"]["right"].pop("state"), "layers[1].mixer.right.state"),
    (lambda r: r["layers"][1]["mlp"]["router"].update(top=7), "layers[1].mlp.router.top"),
    (lambda r: r["layers"][1]["mlp"]["expert"].pop("ff"), "layers[1].mlp.expert.ff"),
    (lambda r: r["layers"][2]["mixer"].pop("kv_rank"), "layers[2].mixer.kv_rank"),
    (lambda r: r["layers"][2]["mixer"]["rot"].update(dims=7), "layers[2].mixer.rot.dims"),
]


@pytest.mark.parametrize("change,field", BROKEN, ids=[f"{n}:{field}" for n, (_, field) in enumerate(BROKEN)])
def test_errors_name_the_key(change, field):
    raw = copy.deepcopy(nu.SMALL["A"])
    change(raw)
    with pytest.raises(ConfigError) as error:
        config_from_dict(raw)
    assert error.value.field == field, str(error.value)


def test_half_split_pairs_are_served_by_reordered_rows():
    """The latent mixer's kernels turn neighbours; the design pairs element i with i + R/2.  Bound weights hold the
    rotated rows in the order (0, R/2, 1, R/2 + 1, ...): turning neighbours of the reordered vector gives the reordered
    turned vector, and a dot product of two vectors reordered alike is the dot product."""
    from leone_amd.parts import MIXERS, POSITIONS, PartSpec
    heads, dim, rot, rank, width = 2, 3, 8, 5, 16
    rope = POSITIONS.build(PartSpec("rope_half_split", {"rotary_dim": rot, "theta": 100.0}))
    part = MIXERS.build(PartSpec("latent_attention", dict(hidden=width, heads=heads, dim=dim, rot_dim=rot, vdim=4, q_rank=None,
                                                          kv_rank=rank, scale=1.0, eps=1e-5, window=None, position="rope", q="q",
                                                          dkv="dkv", dkv_norm="n", uk="uk", uv="uv", o="o")),
                        positions={"rope": rope})
    gen = torch.Generator().manual_seed(0)
    w = {"q": torch.randn(heads * (dim + rot), width, generator=gen), "dkv": torch.randn(rank + rot, width, generator=gen),
         "n": torch.ones(rank), "uk": torch.randn(heads * dim, rank, generator=gen), "uv": torch.randn(heads * 4, rank, generator=gen),
         "o": torch.randn(width, heads * 4, generator=gen)}
    part.bind(dict(w))
    order = [0, 4, 1, 5, 2, 6, 3, 7]
    q_rows = part.w_down[:heads * (dim + rot)]
    for h in range(heads):
        at = h * (dim + rot)
        assert torch.equal(q_rows[at:at + dim], w["q"][at:at + dim])
        assert torch.equal(q_rows[at + dim:at + dim + rot], w["q"][at + dim:at + dim + rot][order])
    kv_rows = part.w_down[heads * (dim + rot):]
    assert torch.equal(kv_rows[:rank], w["dkv"][:rank]) and torch.equal(kv_rows[rank:], w["dkv"][rank:][order])
    x = torch.randn(5, 1, rot, generator=gen, dtype=torch.float64)
    positions = [0, 3, 9, 11, 40]
    want = plain.rotate_halves(x, positions, rot, 100.0)[..., order]
    assert torch.allclose(plain.rotate_neighbours(x[..., order], positions, rot, 100.0), want, atol=1e-12)


def test_plain_pieces_agree_with_one_another():
    """The plain model walked whole and its prefix agree (causality); the convolution's first rows see zeros; the
    router's weights are the softmax over the winners; the state-space walk with no decay and unit steps is a running
    sum of outer products."""
    raw = nu.SMALL["A"]
    weights = {k: v.float() for k, v in nu.make_weights(raw, 3, torch.float32).items()}
    tokens = list(range(3, 50))
    whole = plain.forward(raw, weights, tokens)
    assert torch.allclose(plain.forward(raw, weights, tokens[:23]), whole[:23], atol=1e-9)
    assert float(whole.abs().max()) < raw["logit_softcap"]
    u = torch.arange(12, dtype=torch.float64).view(6, 2) + 1.0
    taps = torch.tensor([[1.0, 10.0, 100.0], [0.0, 0.0, 1.0]], dtype=torch.float64)
    y = plain.short_convolution(u, taps)
    assert y[0].tolist() == [100.0 * 1, 2.0] and y[1].tolist() == [10.0 * 1 + 100.0 * 3, 4.0]
    assert y[5].tolist() == [1.0 * 7 + 10.0 * 9 + 100.0 * 11, 12.0]
    gen = torch.Generator().manual_seed(0)
    h, router = torch.randn(30, 16, generator=gen, dtype=torch.float64), torch.randn(9, 16, generator=gen, dtype=torch.float64)
    chosen, weight = plain.route(h, router, 3)
    logits = h @ router.T
    for row in range(30):
        best = sorted(range(9), key=lambda e: -float(logits[row, e]))[:3]
        assert chosen[row].tolist() == best
        e = torch.exp(logits[row, best])
        assert torch.allclose(weight[row], e / e.sum())
    assert plain.query_temperature([0, 6, 7, 15, 16], {"coef": 2.0, "every": 8}).tolist() == \
        pytest.approx([1.0, 1.0, 1.0 + 2.0 * math.log(2.0), 1.0 + 2.0 * math.log(3.0), 1.0 + 2.0 * math.log(3.0)])
