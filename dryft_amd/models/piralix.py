"""Piralix: from ``PiralixConfig`` to a model plan.

A decoder whose layers differ from one another. Each layer has one mixer (grouped-query attention with a
capped score, a sink and an output gate; a matrix memory; or a gated linear recurrence) and, optionally, a
clamped gated feed-forward, every branch between two RMS norms on a float32 residual stream
(``x <- x + norm_b(branch(norm_a(x)))``). A run of layers may be looped: it runs ``times`` times with the same
weights, each pass with cache lines of its own; a pass begins by adding one learned vector per pass to the
stream and, from the second pass on, the embedding's output once more. A final norm, and the embedding table
as the output head.

What the design fixes rather than the file: the feed-forward's sigmoid slope 1.702, the recurrence's decay
scale 8 and the matrix memory's ``dim^-1/2`` and ``1e-6`` (defaults of those parts), attention weights in float.
Checkpoint names: ``embed``, ``final.norm``, ``loop.step``, and per layer ``l<i>.norm1``, ``norm1b``, ``norm2``,
``norm2b``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""

from __future__ import annotations

from ..config.piralix import PiralixConfig
from ..config.plan import LayerSpec, ModelPlan, PartSpec, Run
from . import register_architecture


def _norm(cfg: PiralixConfig, name: str) -> PartSpec:
    return PartSpec("stream_rmsnorm", dict(size=cfg.width, eps=cfg.norm_eps), {"weight": name})


def _mixer(cfg: PiralixConfig, kind: str, m: dict, p: str, positions: dict[str, PartSpec]) -> PartSpec:
    if kind == "attention":
        rot, name = m["rot"], None
        if rot is not None:
            spec = PartSpec("pair_rotary", dict(dims=rot.dims, base=rot.base, scaling=dict(rot.scaling) if rot.scaling else None))
            name = next((n for n, s in positions.items() if s == spec), None)     # layers with equal rotations share tables
            if name is None:
                name = f"rotary{len(positions)}"
                positions[name] = spec
        return PartSpec(
            "gqa_attention",
            dict(hidden_size=cfg.width, num_heads=m["heads"], num_kv_heads=m["kv_heads"], head_dim=m["dim"],
                 value_dim=m["vdim"], positions=name, scale=m["scale"], softcap=m["softcap"], sink=True,
                 output_gate=True, float_weights=True),
            {"q_proj": p + "q", "k_proj": p + "k", "v_proj": p + "v", "g_proj": p + "g", "o_proj": p + "o",
             "sink": p + "sink"})
    if kind == "mlstm":
        return PartSpec(
            "matrix_memory",
            dict(hidden_size=cfg.width, num_heads=m["heads"], key_dim=m["dim"], value_dim=m["vdim"],
                 gate_cap=m["gate_cap"], norm_eps=cfg.norm_eps),
            {"q_proj": p + "q", "k_proj": p + "k", "v_proj": p + "v", "g_proj": p + "g", "o_proj": p + "o",
             "out_norm": p + "norm", "i_proj": p + "i", "i_bias": p + "i.b", "f_proj": p + "f", "f_bias": p + "f.b"})
    return PartSpec(
        "gated_linear_recurrence",
        dict(hidden_size=cfg.width, width=m["width"], blocks=m["blocks"], taps=m["conv"]),
        {"y_proj": p + "y", "y_bias": p + "y.b", "x_proj": p + "x", "x_bias": p + "x.b", "conv": p + "conv",
         "conv_bias": p + "conv.b", "gate_a": p + "ra", "gate_a_bias": p + "ra.b", "gate_i": p + "ri",
         "gate_i_bias": p + "ri.b", "lam": p + "lam", "o_proj": p + "o"})


def piralix_plan(cfg: PiralixConfig) -> ModelPlan:
    positions: dict[str, PartSpec] = {}
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        parts = {"mixer_norm": _norm(cfg, p + "norm1"),
                 "mixer": _mixer(cfg, layer.type, layer.mixer_dict(), p + "mix.", positions),
                 "mixer_post_norm": _norm(cfg, p + "norm1b")}
        if layer.mlp is None:
            layers.append(LayerSpec("sandwich_mixer", parts))
            continue
        mlp = dict(layer.mlp)
        parts.update({
            "ffn_norm": _norm(cfg, p + "norm2"),
            "ffn": PartSpec("clamped_glu", dict(hidden_size=cfg.width, intermediate_size=mlp["ff"], limit=mlp["limit"]),
                            {"gate_proj": p + "mlp.gate", "up_proj": p + "mlp.up", "down_proj": p + "mlp.down"}),
            "ffn_post_norm": _norm(cfg, p + "norm2b")})
        layers.append(LayerSpec("sandwich", parts))
    # the schedule: layers before the loop, the looped run once per pass (each pass with cache lines of its own,
    # its first run entering through the pass entry), the layers after it
    n = len(cfg.layers)
    order: list[tuple[int, tuple[str, int] | None]] = []
    stream_parts = {}
    if cfg.loop is None:
        order = [(i, None) for i in range(n)]
    else:
        lp = cfg.loop
        stream_parts["loop"] = PartSpec("pass_entry", dict(passes=lp.times, size=cfg.width), {"steps": "loop.step"})
        order += [(i, None) for i in range(lp.start)]
        for t in range(lp.times):
            order += [(i, ("loop", t) if i == lp.start else None) for i in range(lp.start, lp.stop)]
        order += [(i, None) for i in range(lp.stop, n)]
    schedule = tuple(Run(layer, line, True, enter) for line, (layer, enter) in enumerate(order))
    return ModelPlan(
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        embedding=PartSpec("token_embedding", dict(vocab_size=cfg.vocab, hidden_size=cfg.width), {"weight": "embed"}),
        layers=tuple(layers),
        schedule=schedule,
        final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab, hidden_size=cfg.width), {"weight": "embed"}),
        positions=positions,
        stream_parts=stream_parts,
        max_positions=None,
    )


register_architecture(PiralixConfig.architecture, PiralixConfig, piralix_plan)
