"""Piralix on the GPU against the plain implementation (float64), in float32 and bfloat16: each new mechanism alone,
then whole models of four configurations through the step function (whole prompts, portions down to two tokens,
one token at a time, unequal batches, slots used again, long decoding), greedy generation through the entry point
with captured steps, and the trace program."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import collect_positions, trace_batches
from piralix_cases import CASES, SCALING, double, tensors_for, write_dir
from plain import piralix_plain as P

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}
# |got - want| (root mean square over a row, the row's mean difference taken off) over the root mean square of the
# rows wanted: float32 rounding through a dozen layer runs; bfloat16 activations (8 bits) between float32 norms.
# The test models' logits are sharp (a unit-variance embedding as the head): the worst of several hundred bfloat16
# rows comes to 0.045 of the logits' size, while a lost state, a missed key or a sink left out moves rows by 0.2 and
# more (the tests below that build such cases say so).
TOL = {"float32": 2e-4, "bfloat16": 7e-2}
# One mixer: its projections are rounded to 8 bits, and the worst row of a few hundred is taken (a read-out whose
# normaliser is small magnifies the rounding of q and k).
MIXER_TOL = {"float32": 3e-5, "bfloat16": 4e-2}


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return float(d.pow(2).mean(-1).sqrt().max() / want.pow(2).mean().sqrt())


# ------------------------------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [60, 256, 1000])
def test_stream_norm_every_combination(dtype, width):
    from dryft_amd.csrc import ops
    T = TORCH[dtype]
    g = torch.Generator().manual_seed(width)
    rows = 7
    x32 = torch.randn(rows, width, generator=g) * 3
    xT = torch.randn(rows, width, generator=g).to(T)
    delta = torch.randn(rows, width, generator=g).to(T)
    parts = torch.randn(3, rows, width, generator=g)
    extra = torch.randn(rows, width, generator=g).to(T)
    vec, wb, w = (torch.randn(width, generator=g) for _ in range(3))
    eps = 1e-5
    for x in (None, x32, xT):
        for d in (None, delta, parts):
            for post in (None, wb):
                for e in (None, extra):
                    for v in (None, vec):
                        if x is None and d is None and e is None:
                            continue
                        want = torch.zeros(rows, width, dtype=torch.float64) if x is None else x.double()
                        if d is not None:
                            dd = d.double().sum(0) if d.dim() == 3 else d.double()
                            want = want + (P.rms(dd, eps) * wb.double() if post is not None else dd)
                        if e is not None:
                            want = want + e.double()
                        if v is not None:
                            want = want + v.double()
                        x_out = torch.empty(rows, width, dtype=torch.float32, device=DEV)
                        y = torch.empty(rows, width, dtype=T, device=DEV)
                        dev = lambda t: None if t is None else t.to(DEV)
                        ops.stream_norm(dev(x), (dev(d), 3) if d is not None and d.dim() == 3 else dev(d), dev(post),
                                        dev(e), dev(v), w.to(DEV), eps, x_out, y, T)
                        assert torch.allclose(x_out.cpu().double(), want, atol=2e-5, rtol=1e-6)
                        yw = P.rms(want, eps) * w.double()
                        assert rel_err(y, yw) <= (1e-6 if dtype == "float32" else 6e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [72, 128, 256])
def test_clamped_glu_part(dtype, hidden):
    """``hidden`` 128 and 256: in bfloat16 steps of up to 64 rows take the product with the unit in its epilogue."""
    from dryft_amd.parts.base import Partials
    from dryft_amd.parts.mlp import ClampedGLU
    T = TORCH[dtype]
    g = torch.Generator().manual_seed(3)
    w = {"gate": 2 * torch.randn(104, hidden, generator=g) / hidden ** 0.5, "up": 2 * torch.randn(104, hidden, generator=g) / hidden ** 0.5,
         "down": torch.randn(hidden, 104, generator=g) / 10}
    w = {k: v.to(T) for k, v in w.items()}
    ffn = ClampedGLU(hidden, 104, limit=0.8)
    ffn.load({k + "_proj": v.to(DEV) for k, v in w.items()})
    for rows in (1, 9, 40, 130):
        h = torch.randn(rows, hidden, generator=g).to(T)
        out = ffn.forward(h.to(DEV), None)
        if isinstance(out, Partials):
            out = out.summed(torch.float32)
        want = P.clamped_glu(h.double(), double(w), {"limit": 0.8})
        assert float((h.double() @ w["gate"].double().T).max()) > 0.8          # the clamp is at work
        assert float((h.double() @ w["up"].double().T).min()) < -0.8
        assert rel_err(out, want) <= MIXER_TOL[dtype]


# ------------------------------------------------------------------------------------------ mixers alone
def run_mixer(mixer, cache, positions, dtype, seqs, cuts):
    """Feed each sequence's rows of hidden states through the mixer in steps cut at ``cuts`` (the same cuts for all;
    a sequence that has ended takes no part)."""
    from dryft_amd.engine.step import BatchBuffers, stage_batch
    from dryft_amd.parts.base import Partials
    T = TORCH[dtype]
    slots = cache.acquire(len(seqs))
    buf = BatchBuffers(1024, 8, DEV)
    outs = [[] for _ in seqs]
    edges = [0] + list(cuts) + [max(len(s) for s in seqs)]
    for a, b in zip(edges[:-1], edges[1:]):
        live = [(i, s[a:b]) for i, s in enumerate(seqs) if len(s[a:b])]
        if not live:
            continue
        q_lens = [len(x) for _, x in live]
        ctx = stage_batch(cache, buf, [slots[i] for i, _ in live], q_lens, [0] * sum(q_lens), T)
        ctx.positions = positions
        h = torch.cat([x for _, x in live]).to(T).to(DEV)
        out = mixer.forward(h, ctx, cache.line(0), True)
        if isinstance(out, Partials):
            out = out.summed(torch.float32)
        cache.end_step([slots[i] for i, _ in live], q_lens)
        at = 0
        for i, x in live:
            outs[i].append(out[at:at + len(x)].float().cpu())
            at += len(x)
    cache.release(slots)
    return [torch.cat(o) for o in outs]


CUTS = ([], list(range(150, 201)), [2, 5, 64, 66, 127], [63, 128])


def mixer_case(kind, m, width, seed):
    """A layer of one mixer cut out of a one-layer configuration: (library part, its plain weights, cache, tables)."""
    from dryft_amd.cache import CacheStore
    from dryft_amd.config.piralix import PiralixConfig
    from dryft_amd.models.piralix import piralix_plan
    from dryft_amd.parts import build_part
    cfg = {"architecture": "Piralix", "vocab": 16, "width": width, "norm": {"eps": 1e-5},
           "layers": [{"type": kind, "mixer": m, "mlp": None}], "loop": None}
    t = tensors_for(cfg, seed)
    plan = piralix_plan(PiralixConfig.from_dict(cfg))
    return cfg, t, plan, build_part


def load_mixer(plan, t, dtype, max_len=256):
    from dryft_amd.cache import CacheStore
    from dryft_amd.parts import build_part
    T = TORCH[dtype]
    spec = plan.layers[0].parts["mixer"]
    part = build_part(spec)
    part.compute_dtype = T
    held = {}
    for logical, (shape, role, _) in part.tensor_specs().items():
        held[logical] = t[spec.tensors[logical]].to(DEV).to(T)
    part.load(held)
    cache = CacheStore({0: part.cache_need()}, max_tokens=64 * 16, n_slots=4, max_len=max_len, dtype=T, device=DEV)
    positions = {}
    for name, ps in plan.positions.items():
        positions[name] = build_part(ps)
        positions[name].prepare(max_len, T, DEV)
    return part, cache, positions


ATTENTION_SHAPES = {
    "rot-part": dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, softcap=15.0,
                     rot={"dims": 8, "base": 10000.0, "scaling": SCALING}),
    "rot-full": dict(heads=8, kv_heads=1, dim=32, vdim=32, scale=0.2, softcap=50.0,
                     rot={"dims": 32, "base": 1e6, "scaling": None}),
    "bare": dict(heads=3, kv_heads=3, dim=20, vdim=12, scale=0.25, softcap=None, rot=None),
    # the widths of real models' heads: half of each head rotated with scaled frequencies; a head of 64 without a cap
    "head-128": dict(heads=4, kv_heads=2, dim=128, vdim=128, scale=128 ** -0.5, softcap=50.0,
                     rot={"dims": 64, "base": 1e6, "scaling": {"factor": 8.0, "original": 128, "fast": 32.0, "slow": 1.0}}),
    "head-64": dict(heads=2, kv_heads=2, dim=64, vdim=64, scale=0.125, softcap=None,
                    rot={"dims": 64, "base": 10000.0, "scaling": None}),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", sorted(ATTENTION_SHAPES))
def test_attention_alone(dtype, shape):
    m = ATTENTION_SHAPES[shape]
    cfg, t, plan, _ = mixer_case("attention", m, 64, seed=len(shape))
    part, cache, positions = load_mixer(plan, t, dtype)
    g = torch.Generator().manual_seed(11)
    seqs = [torch.randn(n, 64, generator=g).to(TORCH[dtype]).float() for n in (201, 9, 70)]
    w = double(P.sub(t, "l0.mix."))
    want = [P.attention(s.double(), w, m, 1e-5)[0] for s in seqs]
    for cuts in CUTS:
        for got, ref in zip(run_mixer(part, cache, positions, dtype, seqs, cuts), want):
            assert rel_err(got, ref) <= MIXER_TOL[dtype], (shape, cuts[:3])


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_far_key_and_sink_show(dtype):
    """Weights and inputs made so that one key far back takes most of the weight of the last rows, across two page
    borders, in a prompt and in decoding; and so that leaving the sink out, or the cap, would change the output by
    far more than the tolerance."""
    m = dict(heads=2, kv_heads=1, dim=16, vdim=16, scale=0.5, softcap=8.0, rot=None)
    cfg, t, plan, _ = mixer_case("attention", m, 32, seed=2)
    t["l0.mix.q"] = torch.cat([t["l0.mix.k"], t["l0.mix.k"]])            # q . k is large where the inputs agree
    t["l0.mix.sink"] = torch.tensor([8.0, 6.0])
    part, cache, positions = load_mixer(plan, t, dtype)
    g = torch.Generator().manual_seed(4)
    h = torch.randn(170, 32, generator=g) * 0.3
    h[3] = torch.randn(32, generator=g) * 0.6
    h[150:] = h[3] + 0.1 * torch.randn(20, 32, generator=g)               # the last rows ask for key 3
    h = h.to(TORCH[dtype]).float()
    w = double(P.sub(t, "l0.mix."))
    want, _ = P.attention(h.double(), w, m, 1e-5)
    no_sink, _ = P.attention(h.double(), {**w, "sink": w["sink"] - 50}, m, 1e-5)
    no_cap, _ = P.attention(h.double(), w, {**m, "softcap": None}, 1e-5)
    near_only, _ = P.attention(h[4:].double(), w, m, 1e-5)
    assert rel_err(no_sink[150:], want[150:]) > 0.1 and rel_err(no_cap[150:], want[150:]) > 0.1
    assert rel_err(near_only[146:], want[150:]) > 0.1                     # key 3 matters to rows 150..
    for cuts in ([], list(range(140, 170)), [64, 128], [149, 151]):
        got = run_mixer(part, cache, positions, dtype, [h], cuts)[0]
        assert rel_err(got[150:], want[150:]) <= MIXER_TOL[dtype], cuts[:3]


MEMORY_SHAPES = {"narrow": dict(heads=2, dim=16, vdim=24, gate_cap=8.0), "one": dict(heads=1, dim=40, vdim=8, gate_cap=15.0),
                 "wide": dict(heads=3, dim=24, vdim=72, gate_cap=12.0), "deep": dict(heads=1, dim=200, vdim=130, gate_cap=10.0),
                 # a real model's head: four runs of value columns, two tiles of key features a wave; and the widest key
                 "head-128": dict(heads=2, dim=128, vdim=256, gate_cap=15.0), "key-256": dict(heads=1, dim=256, vdim=64, gate_cap=15.0)}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", sorted(MEMORY_SHAPES))
def test_matrix_memory_alone(dtype, shape):
    m = MEMORY_SHAPES[shape]
    cfg, t, plan, _ = mixer_case("mlstm", m, 64, seed=len(shape))
    part, cache, positions = load_mixer(plan, t, dtype)
    g = torch.Generator().manual_seed(12)
    seqs = [torch.randn(n, 64, generator=g).to(TORCH[dtype]).float() for n in (201, 9, 70)]
    w = double(P.sub(t, "l0.mix."))
    want = [P.mlstm(s.double(), w, m, 1e-5)[0] for s in seqs]
    for cuts in CUTS:
        for got, ref in zip(run_mixer(part, cache, positions, dtype, seqs, cuts), want):
            assert rel_err(got, ref) <= MIXER_TOL[dtype], (shape, cuts[:3])


@pytest.mark.parametrize("dtype", DTYPES)
def test_matrix_memory_keeps_an_early_token(dtype):
    """Forget gates near one and a single open input gate: what the memory gives hundreds of tokens later is what
    token 2 wrote, so a state that is dropped, reset or carried in 16 bits shows."""
    m = dict(heads=1, dim=16, vdim=16, gate_cap=20.0)
    cfg, t, plan, _ = mixer_case("mlstm", m, 32, seed=9)
    t["l0.mix.f"] = torch.zeros(1, 32)
    t["l0.mix.f.b"] = torch.tensor([12.0])                                  # log f = -6e-6 a token
    t["l0.mix.i.b"] = torch.tensor([-12.0])
    t["l0.mix.i"] = torch.zeros(1, 32)
    t["l0.mix.i"][0, 0] = 6.0                                              # the input gate opens on feature 0
    part, cache, positions = load_mixer(plan, t, dtype, max_len=512)
    g = torch.Generator().manual_seed(5)
    h = torch.randn(400, 32, generator=g)
    h[:, 0] = -1.0
    h[2, 0] = 3.0
    h = h.to(TORCH[dtype]).float()
    w = double(P.sub(t, "l0.mix."))
    want, _ = P.mlstm(h.double(), w, m, 1e-5)
    lost = h.clone()
    lost[2, 0] = -1.0
    assert rel_err(P.mlstm(lost.double(), w, m, 1e-5)[0][300:], want[300:]) > 0.3
    for cuts in ([], list(range(300, 400)), [2, 3, 64, 257]):
        got = run_mixer(part, cache, positions, dtype, [h], cuts)[0]
        assert rel_err(got[300:], want[300:]) <= MIXER_TOL[dtype], cuts[:3]


RECURRENCE_SHAPES = {"three": dict(width=96, blocks=3, conv=3), "one-tap": dict(width=64, blocks=4, conv=1),
                     "one-block": dict(width=72, blocks=1, conv=2), "five": dict(width=640, blocks=2, conv=5),
                     "blocks-128": dict(width=512, blocks=4, conv=4)}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", sorted(RECURRENCE_SHAPES))
def test_gated_recurrence_alone(dtype, shape):
    m = RECURRENCE_SHAPES[shape]
    cfg, t, plan, _ = mixer_case("rglru", m, 64, seed=len(shape))
    part, cache, positions = load_mixer(plan, t, dtype)
    g = torch.Generator().manual_seed(13)
    seqs = [torch.randn(n, 64, generator=g).to(TORCH[dtype]).float() for n in (201, 9, 70)]
    w = double(P.sub(t, "l0.mix."))
    want = [P.rglru(s.double(), w, m, 1e-5)[0] for s in seqs]
    # cuts shorter than the convolution's memory too: the old inputs move up beside the new ones
    for cuts in CUTS + ([1, 2, 3, 4, 5, 6, 8],):
        for got, ref in zip(run_mixer(part, cache, positions, dtype, seqs, cuts), want):
            assert rel_err(got, ref) <= MIXER_TOL[dtype], (shape, cuts[:3])


# ------------------------------------------------------------------------------------------ whole models
class Model:
    def __init__(self, tmp, name):
        self.name, self.cfg = name, CASES[name]
        self.tensors = tensors_for(self.cfg, seed=ord(name))
        self.dir = write_dir(os.path.join(tmp, name), self.cfg, self.tensors)
        self.vocab = self.cfg["vocab"]
        self._plain, self._engines = {}, {}

    def tokens(self, n, seed=0):
        return [int(x) for x in np.random.default_rng(1000 * seed + n).integers(0, self.vocab, size=n)]

    def plain(self, tokens) -> torch.Tensor:
        key = tuple(tokens)
        if key not in self._plain:
            self._plain[key] = P.forward(self.cfg, double(self.tensors), list(tokens))
        return self._plain[key]

    def engine(self, dtype, **kw):
        from dryft_amd import Engine
        key = (dtype, tuple(sorted(kw.items())))
        if key not in self._engines:
            args = dict(max_batch=4, max_len=320, max_tokens=64 * 24, use_graph=False)
            args.update(kw)
            self._engines[key] = Engine(self.dir, dtype=dtype, **args)
        return self._engines[key]


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    tmp = str(tmp_path_factory.mktemp("piralix"))
    return {name: Model(tmp, name) for name in CASES}


def feed(engine, requests, cuts_of):
    """Each request alone, cut into steps at ``cuts_of(n)``; logits everywhere. Returns {id: [n, vocab]}."""
    from dryft_amd import SeqStep
    out = {}
    for rid, toks in requests.items():
        slot = engine.acquire(1)[0]
        edges = [0] + [c for c in cuts_of(len(toks)) if 0 < c < len(toks)] + [len(toks)]
        got = [engine.step([SeqStep(slot, toks[a:b], list(range(b - a)))]) for a, b in zip(edges[:-1], edges[1:])]
        engine.release([slot])
        out[rid] = torch.cat(got).cpu()
    return out


LENGTHS = [1, 2, 5, 63, 64, 65, 130]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CASES))
def test_whole_prompts_portions_and_single_tokens(models, name, dtype):
    model = models[name]
    engine = model.engine(dtype)
    requests = {f"r{n}": model.tokens(n) for n in LENGTHS}
    for what, cuts_of in (("whole", lambda n: []), ("last tokens one by one", lambda n: list(range(max(1, n - 24), n))),
                          ("portions", lambda n: [2, 4, 7, 64, 66, 129]), ("first tokens one by one", lambda n: [1, 2, 3])):
        got = feed(engine, requests, cuts_of)
        for rid, toks in requests.items():
            assert rel_err(got[rid], model.plain(toks)) <= TOL[dtype], (name, what, rid)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "D"])
def test_layer_by_layer(models, name, dtype):
    """The residual stream after every run of the schedule against the plain one (float32 where the library keeps it)."""
    from dryft_amd import SeqStep
    model = models[name]
    engine = model.engine(dtype)
    toks = model.tokens(37)
    want = []
    P.forward(model.cfg, double(model.tensors), toks, taps=want)
    got = []
    slot = engine.acquire(1)[0]
    engine.step([SeqStep(slot, toks, [36])], tap=lambda i, x: got.append(x.cpu()))
    engine.release([slot])
    assert len(got) == len(want) == len(P.schedule(model.cfg))
    for i, (g, w) in enumerate(zip(got, want)):
        assert g.dtype == torch.float32
        assert rel_err(g, w) <= (2e-5 if dtype == "float32" else 4e-2), (name, i)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CASES))
def test_unequal_batches_and_slots_used_again(models, name, dtype):
    """Three batches one after another in the same slots and pages: unequal prompts start together and decode
    together, the shorter ones end earlier. Against the plain implementation, and against each request alone."""
    from dryft_amd import SeqStep
    model = models[name]
    engine = model.engine(dtype, max_batch=3, max_tokens=64 * 9)
    batches = [{f"b{b}r{n}": (model.tokens(n, seed=b + 1), k) for n, k in sizes}
               for b, sizes in enumerate([[(70, 6), (3, 2), (130, 20)], [(1, 0), (66, 65), (20, 3)], [(129, 1), (64, 10)]])]
    records = list(trace_batches(batches))
    slot_of, outputs = {}, {}
    for rec in records:
        seqs = []
        for e in rec["entries"]:
            if e["id"] not in slot_of:
                slot_of[e["id"]] = engine.acquire(1)[0]
            seqs.append(SeqStep(slot_of[e["id"]], e["tokens"], e["want"]))
        outputs[rec["step"]] = engine.step(seqs).cpu()
        engine.release([slot_of.pop(r) for r in rec["end"]])
    got = collect_positions(records, outputs)
    alone = feed(model.engine(dtype), {rid: toks for b in batches for rid, (toks, _) in b.items()}, lambda n: [])
    for (rid, pos), row in got.items():
        toks = next(b[rid][0] for b in batches if rid in b)
        assert rel_err(row[None], model.plain(toks)[pos][None]) <= TOL[dtype], (name, rid, pos)
        # what else is in the batch, and how the prompt was cut, changes a row by rounding only
        assert rel_err(row[None], alone[rid][pos][None]) <= (2e-5 if dtype == "float32" else TOL[dtype]), (name, rid, pos)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(models, dtype):
    from dryft_amd import SeqStep
    model = models["A"]
    engine = model.engine(dtype)
    toks = model.tokens(300, seed=7)
    want = model.plain(toks)
    slot = engine.acquire(1)[0]
    rows = [engine.step([SeqStep(slot, toks[:2], [1])])]
    for t in toks[2:]:
        rows.append(engine.step([SeqStep(slot, [t], [0])]))
    engine.release([slot])
    assert rel_err(torch.cat(rows).cpu(), want[1:]) <= TOL[dtype]


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(seed, tmp_path):
    """Configurations drawn at random (sizes, head counts, order of layers, rotations, caps, taps, blocks, loops): three
    unequal prompts start together and decode together. float32 must agree with the plain implementation to rounding
    in every row; in bfloat16 the typical row must (single rows of a deep random model, a first token whose q . k is
    near zero for instance, magnify rounding whatever computes them)."""
    import random

    from dryft_amd import Engine, SeqStep
    from piralix_cases import random_config
    cfg = random_config(random.Random(seed))
    tensors = tensors_for(cfg, seed)
    path = write_dir(str(tmp_path / "m"), cfg, tensors)
    g = np.random.default_rng(seed)
    reqs = [[int(x) for x in g.integers(0, cfg["vocab"], size=n)] for n in (1, 37, 150)]
    want = [P.forward(cfg, double(tensors), r) for r in reqs]
    for dtype in DTYPES:
        engine = Engine(path, dtype=dtype, max_batch=4, max_len=256, max_tokens=64 * 16, use_graph=False)
        slots = engine.acquire(3)
        heads = [max(1, len(r) - 6) for r in reqs]
        got = [[] for _ in reqs]
        out = engine.step([SeqStep(s, r[:h], list(range(h))) for s, r, h in zip(slots, reqs, heads)]).cpu()
        at = 0
        for i, h in enumerate(heads):
            got[i].append(out[at:at + h])
            at += h
        for k in range(6):
            live = [(i, s) for i, s in enumerate(slots) if heads[i] + k < len(reqs[i])]
            if live:
                out = engine.step([SeqStep(s, [reqs[i][heads[i] + k]], [0]) for i, s in live]).cpu()
                for j, (i, _) in enumerate(live):
                    got[i].append(out[j:j + 1])
        engine.release(slots)
        for mine, ref in zip(got, want):
            mine = torch.cat(mine).double()
            d = mine - ref
            d = d - d.mean(-1, keepdim=True)
            rows = d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()
            if dtype == "float32":
                assert float(rows.max()) <= TOL[dtype], (seed, cfg["layers"])
            else:
                assert float(rows.median()) <= 0.1 and float(rows.max()) <= 1.0, (seed, float(rows.median()), float(rows.max()))


def plain_greedy(model, prompt, n):
    toks, out, logits = list(prompt), [], []
    for _ in range(n):
        row = P.forward(model.cfg, double(model.tensors), toks)[-1]
        logits.append(row)
        out.append(int(row.argmax()))
        toks.append(out[-1])
    return out, logits


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_greedy_generation_through_the_entry_point(models, name, dtype):
    """``Engine.generate`` with captured steps: the scheduler, the sampler and the graphs serve this design as they
    serve the others. Every token is the plain loop's, or one the plain logits leave within the tolerance of the best."""
    model = models[name]
    prompts = [model.tokens(n, seed=3) for n in (5, 17, 2)]
    for use_graph in (True, False):
        engine = model.engine(dtype, max_batch=4, max_len=64, max_tokens=64 * 4, use_graph=use_graph)
        got = engine.generate_all(prompts, 8)
        assert [len(g) for g in got] == [8, 8, 8]
        for prompt, mine in zip(prompts, got):
            want, logits = plain_greedy(model, prompt, 8)
            for t in range(8):
                if mine[t] != want[t]:
                    spread = float(logits[t].max() - logits[t].min())
                    assert float(logits[t].max() - logits[t][mine[t]]) <= 4 * TOL[dtype] * spread, (name, t)
                    break
    # a second generation in the same engine reuses slots, states and captured steps, and repeats the first token for token
    engine = model.engine(dtype, max_batch=4, max_len=64, max_tokens=64 * 4, use_graph=True)
    first = engine.generate_all(prompts, 8)
    assert engine.generate_all(prompts, 8) == first


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_program(models, dtype, tmp_path):
    model = models["C"]
    batches = [{f"r{n}": (model.tokens(n, seed=9), k) for n, k in [(40, 5), (2, 1), (90, 12)]}, {"s": (model.tokens(65, seed=2), 64)}]
    records = list(trace_batches(batches))
    live = max(sum(len(t) for t, _ in b.values()) for b in batches)
    out_dir = str(tmp_path / "out")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model.dir, "--dtype", dtype, "--out", out_dir,
           "--max-tokens", str(live)]
    proc = subprocess.run(cmd, input="".join(json.dumps(r) + "\n" for r in records), capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split("\n")[:-1] == [f"done {r['step']}" for r in records]
    outputs = {}
    for r in records:
        n_want = sum(len(e["want"]) for e in r["entries"])
        if n_want:
            outputs[r["step"]] = torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{r['step']}.f32"), dtype="<f4").reshape(n_want, model.vocab))
    for (rid, pos), row in collect_positions(records, outputs).items():
        toks = next(b[rid][0] for b in batches if rid in b)
        assert rel_err(row[None], model.plain(toks)[pos][None]) <= TOL[dtype], (rid, pos)
