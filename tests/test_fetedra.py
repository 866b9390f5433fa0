"""Fetedra without a GPU: the configuration reader, the plan's tensor names, a rank that only the checkpoint gives,
and the plain implementation against itself (a prompt whole, in portions and token by token) and against
hand-made cases of its router and window."""

import random

import pytest
import torch

from fetedra_cases import CASES, config, dense, double, latent, moe, random_config, tensors_for, with_mlp, wkv, write_dir
from plain import fetedra_plain as P


def build(cfg):
    from dryft_amd.config.fetedra import FetedraConfig
    from dryft_amd.engine.model import DecoderModel
    from dryft_amd.models import resolve_architecture
    arch = resolve_architecture(cfg)
    assert arch.config_class is FetedraConfig
    return DecoderModel(arch.plan(arch.config_class.from_dict(cfg)), torch.float32, "cpu")


@pytest.mark.parametrize("name", sorted(CASES))
def test_plan_names_every_tensor(name):
    cfg = CASES[name]
    model = build(cfg)
    specs = {s.name: s.shape for s in model.tensor_specs()}
    tensors = tensors_for(cfg, 1)
    assert set(specs) == set(tensors)
    for n, shape in specs.items():
        assert len(shape) == tensors[n].dim() and all(a in (-1, b) for a, b in zip(shape, tensors[n].shape)), n
    needs = model.cache_needs()
    assert len(needs) == len(cfg["layers"])


def test_random_configurations_are_read():
    for seed in range(30):
        cfg = random_config(random.Random(seed))
        model = build(cfg)
        assert {s.name for s in model.tensor_specs()} == set(tensors_for(cfg, seed))


def test_configuration_problems_come_in_one_error():
    from dryft_amd.config.base import ConfigError
    from dryft_amd.config.fetedra import FetedraConfig
    bad = config(64, 100, 9, [with_mlp(wkv(2, 16), {"kind": "sparse"}),
                              with_mlp(latent(2, 16, 8, 16, 8, 16, rot_dims=10), moe(6, 4, 8, groups=(4, 2)))])
    del bad["norm"]
    with pytest.raises(ConfigError) as e:
        FetedraConfig.from_dict(bad)
    text = str(e.value)
    for piece in ("streams", "norm", "layers[0].mlp.kind", "layers[1].mixer.rot.dims", "layers[1].mlp.router.groups.count"):
        assert piece in text, piece
    good = FetedraConfig.from_dict(CASES["A"])
    assert FetedraConfig.from_dict(good.to_dict()) == good


def test_a_rank_only_the_checkpoint_gives(tmp_path):
    """The width of the decay's inner projection is in no configuration key: the loader takes what the file holds,
    the part checks that its two matrices agree, and random weights need the key ``decay_rank``."""
    from dryft_amd.weights.loader import WeightError, load_tensors
    from dryft_amd.weights.random_init import random_tensors
    cfg = config(32, 50, 2, [wkv(2, 8)])
    model = build(cfg)
    tensors = tensors_for(cfg, 0, decay_rank=5)
    path = write_dir(str(tmp_path / "m"), cfg, tensors)
    held = load_tensors(path, model.tensor_specs(), torch.float32)
    assert held["l0.mix.w1"].shape == (5, 32) and held["l0.mix.w2"].shape == (16, 5)
    model.load(dict(held))
    tensors["l0.mix.w2"] = torch.zeros(16, 4)
    bad = write_dir(str(tmp_path / "bad"), cfg, tensors)
    with pytest.raises(ValueError, match="rank"):
        build(cfg).load(load_tensors(bad, model.tensor_specs(), torch.float32))
    tensors["l0.mix.w2"] = torch.zeros(17, 5)
    with pytest.raises(WeightError):
        load_tensors(write_dir(str(tmp_path / "worse"), cfg, tensors), model.tensor_specs(), torch.float32)
    with pytest.raises(ValueError, match="checkpoint"):
        random_tensors(model.tensor_specs(), 0)
    cfg["layers"][0]["mixer"]["decay_rank"] = 3
    drawn = random_tensors(build(cfg).tensor_specs(), 0)
    assert drawn["l0.mix.w1"].shape == (3, 32)
    assert float(drawn["l0.norm1"].abs().max()) == 0 and torch.equal(drawn["l0.hc1.mix"].float(), torch.eye(2))


@pytest.mark.parametrize("name", sorted(CASES))
def test_plain_prompt_equals_portions_equals_single_tokens(name):
    cfg = CASES[name]
    t = double(tensors_for(cfg, 2))
    toks = torch.randint(0, cfg["vocab"], (90,), generator=torch.Generator().manual_seed(1))
    whole, _ = P.forward(cfg, t, toks)
    for cuts in ([1, 2, 64, 66], list(range(1, 90))):
        state, rows = None, []
        for a, b in zip([0] + cuts, cuts + [90]):
            out, state = P.forward(cfg, t, toks[a:b], state)
            rows.append(out)
        assert torch.allclose(torch.cat(rows), whole, atol=1e-9)


def test_plain_router_by_hand():
    """Twelve experts in four groups of three, two groups kept, three chosen; scores picked so that the best single
    expert sits in a group that loses, and all choice scores are negative."""
    s = torch.tensor([[.50, .10, .10, .40, .39, .10, .30, .28, .29, .45, .05, .05]], dtype=torch.float64)
    w = {"router": torch.eye(12, dtype=torch.float64), "correction": torch.full((12,), -1.0, dtype=torch.float64)}
    z = torch.log(s / (1 - s))
    c = moe(12, 3, 8, groups=(4, 2), scale=2.0)
    # group scores (two best, each minus one): -1.40, -1.21, -1.41, -1.50 -> groups 1 and 0
    chosen, weights = P.route(z, w, c)
    assert chosen.tolist() == [[0, 3, 4]]
    assert torch.allclose(weights, torch.tensor([[.50, .40, .39]], dtype=torch.float64) / 1.29 * 2.0)
    # without groups the three best win
    chosen, _ = P.route(z, w, moe(12, 3, 8))
    assert chosen.tolist() == [[0, 9, 3]]


def test_plain_window_by_hand():
    """A window of three: row 5 sees keys 3, 4, 5 and nothing else, whatever their scores."""
    layer = latent(1, 4, 2, 4, 4, 4, window=3)
    cfg = config(8, 10, 1, [layer])
    t = double(tensors_for(cfg, 5))
    w = P.part(t, "l0.mix.")
    h = torch.randn(6, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    out, _ = P.latent_attention(h, w, layer["mixer"], 1e-5)
    moved = h.clone()
    moved[:3] += 1.0
    again, _ = P.latent_attention(moved, w, layer["mixer"], 1e-5)
    assert torch.allclose(out[5], again[5]) and not torch.allclose(out[4], again[4])
