"""Fetedra: from ``FetedraConfig`` to a model plan.

A decoder on several copies of a float32 residual stream ("hyper-connections"): every sublayer reads a weighted
sum of the copies through an RMS norm whose weight is stored as its distance from one, and its output goes back to
every copy with a weight of its own while the copies are mixed with one another by a small matrix. Each layer has
one mixer (``wkv``: token-shifted projections into a matrix state per head with a data-dependent decay; or
``latent_attention``: queries, keys and values through low-rank latents, one rotated key part shared by all heads,
a sliding window, a sink and a gate per head) and, optionally, a feed-forward (gated dense, or routed experts with
a shared one). At the end the copies are summed and normed; the head is the embedding table times ``logit_scale``.

What the design fixes rather than the file: the experts' sigmoid slope 1.702, the two best choice scores that make
a group's score, the ``1e-20`` under the routing weights (defaults of those parts). Checkpoint names: ``embed``,
``final.norm``, and per layer ``l<i>.norm1``, ``norm2``, ``l<i>.hc1.{in,out,mix}``, ``hc2.*``, ``l<i>.mix.*``,
``l<i>.mlp.*``.
"""

from __future__ import annotations

from ..config.fetedra import FetedraConfig
from ..config.plan import LayerSpec, ModelPlan, PartSpec, Run
from . import register_architecture


def _norm(cfg: FetedraConfig, name: str, scale: float = 1.0) -> PartSpec:
    return PartSpec("stream_rmsnorm", dict(size=cfg.width, eps=cfg.norm_eps, offset=1.0, scale=scale), {"weight": name})


def _route(cfg: FetedraConfig, p: str) -> PartSpec:
    return PartSpec("stream_route", dict(streams=cfg.streams), {"read": p + "in", "write": p + "out", "mix": p + "mix"})


def _mixer(cfg: FetedraConfig, kind: str, m: dict, p: str, positions: dict[str, PartSpec]) -> PartSpec:
    if kind == "wkv":
        return PartSpec(
            "wkv", dict(hidden_size=cfg.width, num_heads=m["heads"], head_dim=m["dim"], decay_rank=m.get("decay_rank"),
                        norm_eps=cfg.norm_eps),
            {"mu_r": p + "mu.r", "mu_k": p + "mu.k", "mu_v": p + "mu.v", "mu_g": p + "mu.g", "mu_w": p + "mu.w",
             "r_proj": p + "r", "k_proj": p + "k", "v_proj": p + "v", "g_proj": p + "g", "decay_down": p + "w1",
             "decay_up": p + "w2", "decay_bias": p + "w0", "bonus": p + "u", "out_norm": p + "norm", "o_proj": p + "o"})
    rot, name = m["rot"], None
    if rot["dims"]:
        spec = PartSpec("half_rotary", dict(dims=rot["dims"], base=rot["base"]))
        name = next((n for n, s in positions.items() if s == spec), None)     # layers with equal rotations share tables
        if name is None:
            name = f"rotary{len(positions)}"
            positions[name] = spec
    return PartSpec(
        "latent_attention",
        dict(hidden_size=cfg.width, num_heads=m["heads"], head_dim=m["dim"], rot_dim=m["rot_dim"], value_dim=m["vdim"],
             q_rank=m["q_rank"], kv_rank=m["kv_rank"], scale=m["scale"], positions=name,
             window=m["mask"]["size"] if m["mask"] else None, norm_eps=cfg.norm_eps),
        {"q_down": p + "dq", "q_norm": p + "dq.norm", "q_up": p + "uq", "kv_down": p + "dkv", "kv_norm": p + "dkv.norm",
         "k_up": p + "uk", "v_up": p + "uv", "sink": p + "sink", "g_proj": p + "g", "o_proj": p + "o"})


def _mlp(cfg: FetedraConfig, mlp: dict, p: str) -> PartSpec:
    if mlp["kind"] == "dense":
        return PartSpec("swiglu", dict(hidden_size=cfg.width, intermediate_size=mlp["ff"]),
                        {"gate_proj": p + "gate", "up_proj": p + "up", "down_proj": p + "down"})
    r, shared = mlp["router"], mlp["shared"]
    names = {"router": p + "router", "correction": p + "correction"}
    for e in range(r["experts"]):
        for t in ("gate", "up", "down"):
            names[f"e{e}_{t}"] = f"{p}e{e}.{t}"
    if shared:
        names.update({"shared_gate": p + "shared.gate", "shared_up": p + "shared.up", "shared_down": p + "shared.down",
                      "shared_weight": p + "shared.sg"})
    return PartSpec(
        "routed_experts",
        dict(hidden_size=cfg.width, experts=r["experts"], top=r["top"], intermediate_size=mlp["expert"]["ff"],
             limit=mlp["expert"]["limit"], route_scale=r["scale"],
             groups=(r["groups"]["count"], r["groups"]["keep"]) if r["groups"] else None,
             shared=(shared["ff"], shared["limit"]) if shared else None),
        names)


def fetedra_plan(cfg: FetedraConfig) -> ModelPlan:
    positions: dict[str, PartSpec] = {}
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        parts = {"mixer_route": _route(cfg, p + "hc1."), "mixer_norm": _norm(cfg, p + "norm1"),
                 "mixer": _mixer(cfg, layer.type, layer.mixer, p + "mix.", positions)}
        if layer.mlp is None:
            layers.append(LayerSpec("hyper_mixer", parts))
            continue
        parts.update({"ffn_route": _route(cfg, p + "hc2."), "ffn_norm": _norm(cfg, p + "norm2"),
                      "ffn": _mlp(cfg, layer.mlp, p + "mlp.")})
        layers.append(LayerSpec("hyper", parts))
    return ModelPlan(
        vocab_size=cfg.vocab,
        hidden_size=cfg.width,
        embedding=PartSpec("token_embedding", dict(vocab_size=cfg.vocab, hidden_size=cfg.width), {"weight": "embed"}),
        layers=tuple(layers),
        schedule=tuple(Run(i, i, True) for i in range(len(layers))),
        # the head's factor rides on the final norm's weight: logits = embed . (norm(x) * (1 + w) * logit_scale)
        final_norm=_norm(cfg, "final.norm", scale=cfg.logit_scale),
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab, hidden_size=cfg.width), {"weight": "embed"}),
        positions=positions,
        max_positions=None,
    )


register_architecture(FetedraConfig.architecture, FetedraConfig, fetedra_plan)
