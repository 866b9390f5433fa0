"""Fetedra on the GPU against the plain implementation (float64), in float32 and bfloat16: each new mechanism alone,
then whole models of three configurations through the step function (whole prompts, portions down to two tokens,
one token at a time, unequal batches, slots used again, long decoding), configurations drawn at random, greedy
generation through the entry point with captured steps, and the trace program."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from fetedra_cases import CASES, config, dense, double, latent, moe, tensors_for, with_mlp, wkv, write_dir
from helpers import collect_positions, trace_batches
from plain import fetedra_plain as P
from test_piralix_gpu import CUTS, MIXER_TOL, TOL, feed, rel_err, run_mixer

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


# ------------------------------------------------------------------------------------------ the copies of the stream
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,width", [(1, 60), (3, 256), (4, 1000), (8, 64)])
def test_stream_copies_every_combination(dtype, n, width):
    from dryft_amd.csrc import ops
    T = TORCH[dtype]
    g = torch.Generator().manual_seed(width + n)
    rows, eps = 7, 1e-5
    copies = torch.randn(n, rows, width, generator=g) * 3
    start = torch.randn(rows, width, generator=g).to(T)
    delta = torch.randn(rows, width, generator=g).to(T)
    parts = torch.randn(3, rows, width, generator=g)
    mix, write, read, w = (torch.randn(s, generator=g) for s in ((n, n), (n,), (n,), (width,)))
    dev = lambda t: None if t is None else t.to(DEV)      # noqa: E731
    for x in (copies, start):
        xs = x.double() if x.dim() == 3 else x.double()[None].expand(n, -1, -1)
        for d in (None, delta, parts):
            want = xs
            if d is not None:
                dd = d.sum(0).to(T).double() if d.dim() == 3 else d.double()
                want = torch.einsum("st,src->trc", mix.double(), xs) + write.double()[:, None, None] * dd
            for rd in (None, read):
                u = want.sum(0) if rd is None else torch.einsum("t,trc->rc", rd.double(), want)
                x_out = torch.empty(n, rows, width, dtype=torch.float32, device=DEV)
                y = torch.empty(rows, width, dtype=T, device=DEV)
                args = (dev(x), n, (dev(d), 3) if d is not None and d.dim() == 3 else dev(d),
                        dev(mix) if d is not None else None, dev(write) if d is not None else None, dev(rd))
                ops.hyper_norm(*args, w.to(DEV), eps, x_out, y, normed=True)
                assert torch.allclose(x_out.cpu().double(), want, atol=3e-5, rtol=1e-6)
                assert rel_err(y, P.rms(u, eps) * w.double()) <= (1e-6 if dtype == "float32" else 6e-3)
                s = torch.empty(rows, width, dtype=torch.float32, device=DEV)
                ops.hyper_norm(*args, None, 0.0, None, s, normed=False, act=T)
                assert torch.allclose(s.cpu().double(), u, atol=1e-4, rtol=1e-6)


# ------------------------------------------------------------------------------------------ mixers alone
def mixer_case(layer, width, seed, **kw):
    from dryft_amd.config.fetedra import FetedraConfig
    from dryft_amd.models.fetedra import fetedra_plan
    cfg = config(width, 16, 2, [layer])
    t = tensors_for(cfg, seed, **kw)
    return cfg, t, fetedra_plan(FetedraConfig.from_dict(cfg))


def load_mixer(plan, t, dtype, max_len=256):
    from dryft_amd.cache import CacheStore
    from dryft_amd.parts import build_part
    T = TORCH[dtype]
    spec = plan.layers[0].parts["mixer"]
    part = build_part(spec)
    part.compute_dtype = T
    part.load({logical: t[spec.tensors[logical]].to(DEV).to(T) for logical in part.tensor_specs()})
    cache = CacheStore({0: part.cache_need()}, max_tokens=64 * 16, n_slots=4, max_len=max_len, dtype=T, device=DEV)
    positions = {}
    for name, ps in plan.positions.items():
        positions[name] = build_part(ps)
        positions[name].prepare(max_len, T, DEV)
    return part, cache, positions


def sub(t, prefix):
    return double(P.part(t, prefix))


WKV_SHAPES = {"two": (2, 16), "odd": (3, 24), "wide": (1, 80), "head-64": (4, 64), "small": (5, 8), "big": (1, 136)}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", sorted(WKV_SHAPES))
def test_wkv_alone(dtype, shape):
    layer = wkv(*WKV_SHAPES[shape])
    cfg, t, plan = mixer_case(layer, 64, seed=len(shape), decay_rank=len(shape) + 2)
    part, cache, positions = load_mixer(plan, t, dtype)
    g = torch.Generator().manual_seed(12)
    seqs = [torch.randn(n, 64, generator=g).to(TORCH[dtype]).float() for n in (201, 9, 70)]
    w = sub(t, "l0.mix.")
    want = [P.wkv(s.double(), w, layer["mixer"], 1e-5)[0] for s in seqs]
    for cuts in CUTS + ([1, 2, 3, 4, 5, 6, 8],):
        for got, ref in zip(run_mixer(part, cache, positions, dtype, seqs, cuts), want):
            assert rel_err(got, ref) <= MIXER_TOL[dtype], (shape, cuts[:3])


@pytest.mark.parametrize("dtype", DTYPES)
def test_wkv_keeps_an_early_token(dtype):
    """Decays next to one, and keys that are zero but for token 2: what the state gives hundreds of tokens later is
    what token 2 wrote, so a state that is dropped, reset or carried in 16 bits shows. The first token's blend with
    the zeros before it, and the bonus of the token at hand, show in the same way."""
    layer = wkv(1, 16)
    cfg, t, plan = mixer_case(layer, 32, seed=9)
    t["l0.mix.w2"] = torch.zeros_like(t["l0.mix.w2"])
    t["l0.mix.w0"] = torch.full_like(t["l0.mix.w0"], -9.0)                  # w = exp(-exp(-9)): 0.99988 a token
    t["l0.mix.mu.k"] = torch.zeros_like(t["l0.mix.mu.k"])                   # keys read the token itself
    t["l0.mix.k"] = torch.zeros_like(t["l0.mix.k"])
    t["l0.mix.k"][:, 0] = 1.0                                              # and only its feature 0
    part, cache, positions = load_mixer(plan, t, dtype, max_len=512)
    g = torch.Generator().manual_seed(5)
    h = torch.randn(400, 32, generator=g)
    h[:, 0] = 0.0
    h[2, 0] = 3.0
    h = h.to(TORCH[dtype]).float()
    w = sub(t, "l0.mix.")
    want, _ = P.wkv(h.double(), w, layer["mixer"], 1e-5)
    lost = h.clone()
    lost[2, 0] = 0.0
    assert rel_err(P.wkv(lost.double(), w, layer["mixer"], 1e-5)[0][300:], want[300:]) > 0.3
    no_bonus = P.wkv(h.double(), {**w, "u": w["u"] * 0}, layer["mixer"], 1e-5)[0]
    assert rel_err(no_bonus[2:3], want[2:3]) > 0.3
    for cuts in ([], list(range(300, 400)), [2, 3, 64, 257], [1]):
        got = run_mixer(part, cache, positions, dtype, [h], cuts)[0]
        assert rel_err(got[300:], want[300:]) <= MIXER_TOL[dtype], cuts[:3]
        assert rel_err(got[:4], want[:4]) <= MIXER_TOL[dtype], cuts[:3]


LATENT_SHAPES = {
    "cores": latent(4, 16, 16, 32, 40, 48, window=20),                      # keys and values of 32: the matrix cores
    "cores-narrow-values": latent(2, 24, 8, 16, 24, 40, window=70, base=1e6),
    "cores-no-window": latent(3, 8, 8, 16, 16, 24),
    "plain-kernel": latent(3, 20, 6, 12, 18, 28, rot_dims=4, base=500.0),  # keys of 26
    "wide-values": latent(1, 8, 8, 40, 12, 20, window=64),
    "page-and-one": latent(6, 8, 8, 24, 32, 32, window=65),
    "only-itself": latent(2, 16, 16, 32, 16, 64, window=1),
    "head-192": latent(2, 128, 64, 128, 96, 160, window=128, base=1e6, scale=0.03),    # a real model's head
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", sorted(LATENT_SHAPES))
def test_latent_attention_alone(dtype, shape):
    layer = LATENT_SHAPES[shape]
    cfg, t, plan = mixer_case(layer, 64, seed=len(shape))
    part, cache, positions = load_mixer(plan, t, dtype)
    g = torch.Generator().manual_seed(11)
    seqs = [torch.randn(n, 64, generator=g).to(TORCH[dtype]).float() for n in (201, 9, 70)]
    w = sub(t, "l0.mix.")
    want = [P.latent_attention(s.double(), w, layer["mixer"], 1e-5)[0] for s in seqs]
    for cuts in CUTS:
        for got, ref in zip(run_mixer(part, cache, positions, dtype, seqs, cuts), want):
            assert rel_err(got, ref) <= MIXER_TOL[dtype], (shape, cuts[:3])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [None, 20, 64, 65, 130])
def test_latent_attention_edges_far_keys_and_sink_show(dtype, window):
    """A score scale large enough that a row gives most of its weight to one or two keys, wherever they are: then a
    window that is one token off, a key lost behind a page border or a sink left out moves some row by far more than
    the tolerance (the plain implementation with each of those faults shows it), in prompts, portions and decoding.
    Sharp scores also magnify the rounding of q and k to 8 bits: bfloat16 gets twice the usual tolerance here, a
    quarter of what the smallest of the faults moves."""
    tol = {"float32": MIXER_TOL["float32"], "bfloat16": 2 * MIXER_TOL["bfloat16"]}[dtype]
    layer = latent(2, 16, 16, 32, 24, 32, window=window, scale=0.4)
    m = layer["mixer"]
    cfg, t, plan = mixer_case(layer, 32, seed=3)
    t["l0.mix.sink"] = torch.tensor([6.0, 4.0])
    part, cache, positions = load_mixer(plan, t, dtype)
    g = torch.Generator().manual_seed(4)
    h = torch.randn(200, 32, generator=g).to(TORCH[dtype]).float()
    w = sub(t, "l0.mix.")
    want, _ = P.latent_attention(h.double(), w, m, 1e-5)
    if window:
        for off in (-1, 1):
            other = {**m, "mask": {"size": window + off}}
            assert rel_err(P.latent_attention(h.double(), w, other, 1e-5)[0], want) > 0.3
    else:
        near_only, _ = P.latent_attention(h[64:].double(), w, m, 1e-5)
        assert rel_err(near_only[86:], want[150:]) > 0.3                   # keys of the first page matter to rows 150..
    no_sink, _ = P.latent_attention(h.double(), {**w, "sink": w["sink"] - 50}, m, 1e-5)
    assert rel_err(no_sink, want) > 0.3
    for cuts in ([], list(range(120, 200)), [64, 128], [2, 63, 65, 127, 129], [19, 20, 21]):
        got = run_mixer(part, cache, positions, dtype, [h], cuts)[0]
        assert rel_err(got, want) <= tol, cuts[:3]


# ------------------------------------------------------------------------------------------ routed experts alone
def load_ffn(mlp, width, seed, dtype):
    from dryft_amd.config.fetedra import FetedraConfig
    from dryft_amd.models.fetedra import fetedra_plan
    from dryft_amd.parts import build_part
    cfg = config(width, 16, 1, [with_mlp(wkv(1, 8), mlp)])
    t = tensors_for(cfg, seed)
    spec = fetedra_plan(FetedraConfig.from_dict(cfg)).layers[0].parts["ffn"]
    part = build_part(spec)
    part.compute_dtype = TORCH[dtype]
    part.load({logical: t[spec.tensors[logical]].to(DEV).to(TORCH[dtype]) for logical in part.tensor_specs()})
    return part, t


ROUTERS = {
    "groups-of-two": moe(8, 3, 32, limit=1.0, groups=(4, 2), scale=2.0, shared=(40, 1.5)),
    "groups-of-one": moe(6, 2, 24, limit=0.7, groups=(6, 3), shared=(16, 0.5)),
    "no-groups-top-one": moe(5, 1, 20, limit=2.0, scale=1.5),
    "all-chosen": moe(4, 4, 12, limit=1.0, groups=(2, 2)),
    "many": moe(96, 6, 16, limit=1.0, groups=(8, 3), scale=0.5, shared=(24, 1.0)),
    "one-expert": moe(1, 1, 16, shared=(8, 1.0)),
}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(ROUTERS))
def test_routed_experts_alone(dtype, name):
    from dryft_amd.csrc import ops
    from dryft_amd.parts.linear import linear
    mlp = ROUTERS[name]
    part, t = load_ffn(mlp, 72, seed=len(name), dtype=dtype)
    w = sub(t, "l0.mlp.")
    g = torch.Generator().manual_seed(8)
    for rows in (1, 9, 40, 130, 700):
        h = torch.randn(rows, 72, generator=g).to(TORCH[dtype])
        # the router alone: the same experts in the same order, wherever the plain scores are not a rounding apart
        logits = linear(h.to(DEV), part.w_router, out_dtype=torch.float32)
        chosen = torch.empty((rows, part.top), dtype=torch.int32, device=DEV)
        weights = torch.empty((rows, part.top), dtype=torch.float32, device=DEV)
        ops.moe_route(logits, part.correction, part.n_experts, part.groups[0], part.groups[1], part.route_scale, chosen, weights)
        want_chosen, want_weights = P.route(h.double(), w, mlp)
        same = (chosen.cpu().long() == want_chosen).all(-1)
        assert float(same.float().mean()) >= (0.999 if dtype == "float32" else 0.9), name
        assert torch.allclose(weights.cpu().double()[same], want_weights[same], atol=1e-5 if dtype == "float32" else 2e-2)
        out = part.forward(h.to(DEV), None)
        want = P.moe(h.double(), w, mlp)
        if dtype == "float32":
            assert rel_err(out, want) <= MIXER_TOL[dtype], (name, rows)
        else:       # a row whose choice is a rounding apart from the plain one goes through another expert
            d = (out.double().cpu() - want)
            per_row = d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()
            assert float(per_row[same].max()) <= MIXER_TOL[dtype], (name, rows)


def test_routing_masks_groups_out_rather_than_to_zero():
    """All choice scores negative: were the experts of dropped groups given a score of zero instead of dropping
    out, they would win every row."""
    from dryft_amd.csrc import ops
    g = torch.Generator().manual_seed(1)
    rows, E = 64, 12
    logits = torch.randn(rows, E, generator=g)
    correction = torch.full((E,), -2.0)
    chosen = torch.empty((rows, 3), dtype=torch.int32, device=DEV)
    weights = torch.empty((rows, 3), dtype=torch.float32, device=DEV)
    ops.moe_route(logits.to(DEV), correction.to(DEV), E, 4, 2, 1.0, chosen, weights)
    mlp = moe(E, 3, 8, groups=(4, 2))
    w = {"router": torch.eye(E).double(), "correction": correction.double()}
    want, want_w = P.route(logits.double(), w, mlp)
    assert (chosen.cpu().long() == want).all()
    assert torch.allclose(weights.cpu().double(), want_w, atol=1e-6)
    choice = torch.sigmoid(logits.double()) - 2.0
    best = choice.view(rows, 4, 3).topk(2, -1).values.sum(-1).topk(2, -1).indices
    for r in range(rows):
        assert all(int(e) // 3 in best[r].tolist() for e in chosen[r].cpu())


# ------------------------------------------------------------------------------------------ whole models
class Model:
    def __init__(self, tmp, name, cfg=None, seed=None):
        self.name, self.cfg = name, cfg or CASES[name]
        self.tensors = tensors_for(self.cfg, seed=seed if seed is not None else ord(name[0]))
        self.dir = write_dir(os.path.join(tmp, name), self.cfg, self.tensors)
        self.vocab = self.cfg["vocab"]
        self._plain, self._engines = {}, {}

    def tokens(self, n, seed=0):
        return [int(x) for x in np.random.default_rng(1000 * seed + n).integers(0, self.vocab, size=n)]

    def plain(self, tokens) -> torch.Tensor:
        key = tuple(tokens)
        if key not in self._plain:
            self._plain[key] = P.forward(self.cfg, double(self.tensors), torch.tensor(list(tokens)))[0]
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
    tmp = str(tmp_path_factory.mktemp("fetedra"))
    return {name: Model(tmp, name) for name in CASES}


LENGTHS = [1, 2, 5, 63, 64, 65, 130]


def row_errors(got, want):
    d = got.double().cpu() - want
    d = d - d.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()


def close(got, want, dtype, tol=None) -> bool:
    """float32: every row to rounding. bfloat16: the typical row to rounding, and three rows of four within twice
    that: a router whose last chosen expert and the next one are 8 bits apart picks the other one now and then (one
    row in ten with sixteen experts), and such a row, and those after it that see it, go another way. What the
    schedules must get right is pinned in float32, and the bfloat16 kernels one by one above."""
    rows = row_errors(got, want)
    tol = tol or TOL[dtype]
    if dtype == "float32":
        return float(rows.max()) <= tol
    return float(rows.median()) <= tol and float(rows.quantile(0.75)) <= 2 * tol


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
            assert close(got[rid], model.plain(toks), dtype), (name, what, rid)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_layer_by_layer(models, name, dtype):
    """The sum of the copies after every layer against the plain one."""
    from dryft_amd import SeqStep
    model = models[name]
    engine = model.engine(dtype)
    toks = model.tokens(37)
    want = []
    P.forward(model.cfg, double(model.tensors), torch.tensor(toks), taps=want)
    got = []
    slot = engine.acquire(1)[0]
    engine.step([SeqStep(slot, toks, [36])], tap=lambda i, x: got.append(x.cpu()))
    engine.release([slot])
    assert len(got) == len(want) == len(model.cfg["layers"])
    for i, (g, w) in enumerate(zip(got, want)):
        assert g.dtype == torch.float32
        assert close(g, w, dtype, 2e-5 if dtype == "float32" else 4e-2), (name, i)


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
    ids = sorted(got)
    mine = torch.stack([got[k] for k in ids])
    assert close(mine, torch.stack([model.plain(next(b[rid][0] for b in batches if rid in b))[pos] for rid, pos in ids]), dtype)
    # what else is in the batch, and how the prompt was cut, changes a row by rounding only
    assert close(mine, torch.stack([alone[rid][pos] for rid, pos in ids]).double(), dtype)


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
    assert close(torch.cat(rows).cpu(), want[1:], dtype)


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(seed, tmp_path):
    """Configurations drawn at random: three unequal prompts start together and decode together. float32 must agree
    with the plain implementation to rounding in every row; in bfloat16 the typical row must."""
    import random

    from dryft_amd import Engine, SeqStep
    from fetedra_cases import random_config
    cfg = random_config(random.Random(seed))
    tensors = tensors_for(cfg, seed, decay_rank=3 + seed)
    path = write_dir(str(tmp_path / "m"), cfg, tensors)
    g = np.random.default_rng(seed)
    reqs = [[int(x) for x in g.integers(0, cfg["vocab"], size=n)] for n in (1, 37, 150)]
    want = [P.forward(cfg, double(tensors), torch.tensor(r))[0] for r in reqs]
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
            rows = row_errors(torch.cat(mine), ref)
            if dtype == "float32":
                assert float(rows.max()) <= TOL[dtype], (seed, cfg["layers"])
            else:
                assert float(rows.median()) <= 0.1 and float(rows.max()) <= 1.5, (seed, float(rows.median()), float(rows.max()))


def plain_greedy(model, prompt, n):
    toks, out, logits = list(prompt), [], []
    for _ in range(n):
        row = P.forward(model.cfg, double(model.tensors), torch.tensor(toks))[0][-1]
        logits.append(row)
        out.append(int(row.argmax()))
        toks.append(out[-1])
    return out, logits


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CASES))
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


def test_a_long_prompt_in_a_captured_step(models):
    """A prompt long enough for the wkv mixer to cut it into segments, started in a captured step beside a short one
    and a sequence that sits out to fill the step: the same tokens as without captured steps (float32, where the two
    differ by rounding far below any gap between logits)."""
    model = models["A"]
    prompts = [model.tokens(150, seed=4), model.tokens(3, seed=5)]
    got = {}
    for use_graph in (True, False):
        engine = model.engine("float32", max_batch=4, max_len=192, max_tokens=64 * 12, use_graph=use_graph)
        got[use_graph] = engine.generate_all(prompts, 6)
    assert got[True] == got[False]
    want, _ = plain_greedy(model, prompts[0], 6)
    assert got[False][0] == want


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
    got = collect_positions(records, outputs)
    ids = sorted(got)
    want = torch.stack([model.plain(next(b[rid][0] for b in batches if rid in b))[pos] for rid, pos in ids])
    assert close(torch.stack([got[k] for k in ids]), want, dtype)
