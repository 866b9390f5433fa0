"""Piralix without a GPU: the configuration reader, the plan (schedule, cache lines, tensor names), the registry,
and the plain implementation against itself and against hand arithmetic."""

import math

import pytest
import torch

from piralix_cases import CASES, CASE_A, CASE_C, SCALING, double, tensors_for, variant
from plain import piralix_plain as P


def build(cfg):
    from dryft_amd.engine.model import DecoderModel
    from dryft_amd.models import resolve_architecture
    arch = resolve_architecture(cfg)
    plan = arch.plan(arch.config_class.from_dict(cfg))
    return arch, plan, DecoderModel(plan, torch.float32, "cpu")


@pytest.mark.parametrize("name", sorted(CASES))
def test_plan_names_exactly_the_tensors_of_the_configuration(name):
    cfg = CASES[name]
    arch, plan, model = build(cfg)
    assert arch.name == "Piralix"
    want = tensors_for(cfg, 0)
    specs = {s.name: tuple(s.shape) for s in model.tensor_specs()}
    assert specs == {k: tuple(v.shape) for k, v in want.items()}


@pytest.mark.parametrize("name", sorted(CASES))
def test_schedule_follows_the_loop(name):
    cfg = CASES[name]
    _, plan, model = build(cfg)
    runs = P.schedule(cfg)
    assert [r.layer for r in plan.schedule] == [i for i, _ in runs]
    assert [r.enter for r in plan.schedule] == [None if t is None else ("loop", t) for _, t in runs]
    assert [r.cache_line for r in plan.schedule] == list(range(len(runs)))          # a line of its own per run
    assert all(r.writes_cache for r in plan.schedule)
    needs = model.cache_needs()
    for r in plan.schedule:
        kind = cfg["layers"][r.layer]["type"]
        need = needs[r.cache_line]
        assert isinstance(need, dict) == (kind != "attention")


def test_schedule_shapes():
    assert P.schedule(variant(CASE_A, loop=None)) == [(0, None), (1, None), (2, None)]
    assert P.schedule(CASE_A) == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None)]
    assert P.schedule(CASE_C) == [(0, 0), (1, None), (2, None), (3, None), (0, 1), (1, None), (2, None), (3, None)]


def test_configuration_problems_are_collected():
    from dryft_amd.config.base import ConfigError
    from dryft_amd.config.piralix import PiralixConfig
    bad = variant(CASE_A, loop={"start": 2, "stop": 1, "times": 0}, width="wide")
    bad["layers"][0]["mixer"]["kv_heads"] = 3
    bad["layers"][2]["mixer"]["blocks"] = 5
    bad["layers"][1]["type"] = "conv"
    bad["norm"] = {}
    with pytest.raises(ConfigError) as e:
        PiralixConfig.from_dict(bad)
    text = "\n".join(e.value.problems)
    for piece in ("width", "kv_heads", "blocks", "layers[1]", "loop", "norm.eps"):
        assert piece in text, (piece, text)
    cfg = PiralixConfig.from_dict(CASE_A)
    assert PiralixConfig.from_dict(cfg.to_dict()) == cfg


def test_registry_reads_the_single_name():
    from dryft_amd.models import known_architectures, resolve_architecture
    assert "Piralix" in known_architectures()
    assert resolve_architecture({"architecture": "Piralix"}).name == "Piralix"
    assert resolve_architecture({"architectures": ["Piralix"]}).name == "Piralix"


def test_yarn_frequencies_by_hand():
    f, m = P.yarn_frequencies(8, 10000.0, SCALING)
    plain_f = [10000.0 ** (-2 * i / 8) for i in range(4)]
    d = lambda t: 8 * math.log(64 / (2 * math.pi * t)) / (2 * math.log(10000.0))
    lo, hi = max(math.floor(d(8.0)), 0), min(math.ceil(d(1.0)), 7)
    for i in range(4):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0), 1)
        assert abs(float(f[i]) - (plain_f[i] / 4 * ramp + plain_f[i] * (1 - ramp))) < 1e-12
    assert abs(m - (0.1 * math.log(4.0) + 1)) < 1e-12
    f0, m0 = P.yarn_frequencies(8, 10000.0, None)
    assert m0 == 1.0 and torch.allclose(f0, torch.tensor(plain_f, dtype=torch.float64))
    # the library's tables are the same numbers
    from dryft_amd.parts.rope import PairRotaryPositions
    rot = PairRotaryPositions(8, 10000.0, SCALING)
    rot.prepare(50, torch.bfloat16, "cpu")
    a = torch.arange(50, dtype=torch.float64)[:, None] * f[None, :]
    assert rot.cos.dtype == torch.float32 and torch.allclose(rot.cos.double(), a.cos() * m, atol=1e-7)
    assert torch.allclose(rot.sin.double(), a.sin() * m, atol=1e-7)


def test_rotation_turns_neighbours_and_leaves_the_rest():
    x = torch.arange(12, dtype=torch.float64).view(1, 1, 12) + 1
    f = torch.tensor([0.5, 0.25], dtype=torch.float64)
    y = P.rotate_pairs(x, torch.tensor([3]), f, 2.0)
    for i in range(2):
        c, s = 2 * math.cos(3 * f[i]), 2 * math.sin(3 * f[i])
        u, v = float(x[0, 0, 2 * i]), float(x[0, 0, 2 * i + 1])
        assert abs(float(y[0, 0, 2 * i]) - (u * c - v * s)) < 1e-12 and abs(float(y[0, 0, 2 * i + 1]) - (v * c + u * s)) < 1e-12
    assert torch.equal(y[..., 4:], x[..., 4:])


def test_sink_counts_once_and_has_no_value():
    """One token: the only key's weight is exp(s) / (exp(s) + exp(sink)), and the output is that times v."""
    c = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "scale": 1.0, "softcap": None, "rot": None}
    eye = torch.eye(2, dtype=torch.float64)
    w = {"q": eye, "k": eye, "v": eye, "g": torch.zeros(2, 2, dtype=torch.float64), "o": eye,
         "sink": torch.tensor([0.7], dtype=torch.float64)}
    h = torch.tensor([[1.0, 2.0]], dtype=torch.float64)
    out, _ = P.attention(h, w, c, 1e-6)
    p = math.exp(5.0) / (math.exp(5.0) + math.exp(0.7))
    assert torch.allclose(out, 0.5 * p * h)                           # the gate of a zero projection is one half
    c["softcap"] = 2.0
    out, _ = P.attention(h, w, c, 1e-6)
    s = 2.0 * math.tanh(5.0 / 2.0)
    assert torch.allclose(out, 0.5 * math.exp(s) / (math.exp(s) + math.exp(0.7)) * h)


def test_matrix_memory_first_token_by_hand():
    """With m starting at 0: m1 = max(f, i); the memory holds exp(i - m1) k v^T, and a small n . q is held up by exp(-m1)."""
    c = {"heads": 1, "dim": 1, "vdim": 1, "gate_cap": 100.0}
    one, zero = torch.ones(1, 1, dtype=torch.float64), torch.zeros(1, dtype=torch.float64)
    for bi, bf in ((-3.0, 0.0), (2.0, -1.0)):
        w = {"q": one, "k": one, "v": one, "g": torch.zeros(1, 1, dtype=torch.float64), "o": one, "norm": one[0],
             "i": torch.zeros(1, 1, dtype=torch.float64), "i.b": zero + bi, "f": torch.zeros(1, 1, dtype=torch.float64),
             "f.b": zero + bf}
        h = torch.tensor([[0.5]], dtype=torch.float64)
        _, (S, n, m) = P.mlstm(h, w, c, 0.0)
        gi = 100 * math.tanh(bi / 100)
        gf = -math.log1p(math.exp(-100 * math.tanh(bf / 100)))
        m1 = max(gf + 0.0, gi)
        assert abs(float(m) - m1) < 1e-12
        assert abs(float(S) - math.exp(gi - m1) * 0.25) < 1e-12 and abs(float(n) - math.exp(gi - m1) * 0.5) < 1e-12


@pytest.mark.parametrize("name", sorted(CASES))
def test_plain_portions_equal_the_whole(name):
    """The plain implementation fed in portions (down to one token) gives what it gives in one piece: its states
    carry everything."""
    cfg = CASES[name]
    t = double(tensors_for(cfg, 5))
    tokens = torch.randint(0, cfg["vocab"], (23,), generator=torch.Generator().manual_seed(1)).tolist()
    whole = P.forward(cfg, t, tokens)
    for cuts in ([7, 8, 20], list(range(1, 23))):
        states, got = None, []
        edges = [0] + cuts + [23]
        states = [None] * len(P.schedule(cfg))
        for a, b in zip(edges[:-1], edges[1:]):
            got.append(P.forward(cfg, t, tokens[a:b], states))
        assert torch.allclose(torch.cat(got), whole, atol=1e-9)
