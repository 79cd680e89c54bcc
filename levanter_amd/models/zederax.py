"""Zederax as a model description: which parts each layer has and where their tensors come from.

A layer is a parallel block: one RMS norm (``l<i>.norm1``) whose output both the attention (``l<i>.mix.*``) and the
feed-forward (``l<i>.mlp.*``) read, their outputs added to the residual stream together; what the next layer reads is a
weighted sum of the results of all layers so far and of the embedding's output (``l<i>.dwa``). The attention has separate
projections ``q``, ``k``, ``v`` with biases (``.b``), unit-norm queries and keys, a soft cap, a linear distance term with
the slope 2^(-8 (h+1) / heads) for head h, a window, weights mixed over the heads by ``talk``, values blended with the
first blending layer's (``vmix``), a sigmoid gate per head (``g``) and the output projection ``o``. The feed-forward is
``down(act(up h))`` with the polynomial activation of ``act``. The token table ``embed`` is also the head; ``final.norm``
comes before it. Linear weights are stored ``[out, in]``. There is no position table: positions act through the distance
term and the window only.
"""
from __future__ import annotations

import math

from levanter_amd.config.zederax import ZederaxConfig
from levanter_amd.parts.spec import LayerSpec, ModelSpec, PartSpec, PlanEntry, TensorSpec

SLOPE_EXPONENT = 8.0  # head h of H: slope 2^(-8 (h + 1) / H)


def distance_slopes(n_heads: int):
    return [2.0 ** (-SLOPE_EXPONENT * (h + 1) / n_heads) for h in range(n_heads)]


def zederax_model_spec(cfg: ZederaxConfig) -> ModelSpec:
    d, eps = cfg.width, float(cfg.norm_eps)
    n_layers = cfg.n_layers

    def rms_norm(name: str) -> PartSpec:
        return PartSpec("rmsnorm", {"dim": d, "eps": eps, "bias": False}, {"weight": TensorSpec(name, (d,), init="one_plus_normal", std=0.1)},
                        family="norm")

    layers = []
    value_source_seen = False
    for i, layer in enumerate(cfg.layers):
        p, m = f"l{i}", layer["mixer"]
        H, G, hd, vd = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        mask = m.get("mask") or {}
        value_mix = None
        if m.get("v_mix"):
            value_mix = "blend" if value_source_seen else "source"
            value_source_seen = True
        lin = 1.0 / math.sqrt(d)
        tensors = {
            "q.weight": TensorSpec(f"{p}.mix.q", (H * hd, d), std=lin), "q.bias": TensorSpec(f"{p}.mix.q.b", (H * hd,), std=0.3),
            "k.weight": TensorSpec(f"{p}.mix.k", (G * hd, d), std=lin), "k.bias": TensorSpec(f"{p}.mix.k.b", (G * hd,), std=0.3),
            "v.weight": TensorSpec(f"{p}.mix.v", (G * vd, d), std=lin), "v.bias": TensorSpec(f"{p}.mix.v.b", (G * vd,), std=0.3),
            "gate.weight": TensorSpec(f"{p}.mix.g", (H, d), std=lin),
            "talk": TensorSpec(f"{p}.mix.talk", (H, H), init="eye_plus_normal", std=0.3),
            "out.weight": TensorSpec(f"{p}.mix.o", (d, H * vd), std=1.0 / math.sqrt(H * vd)),
        }
        if value_mix == "blend":  # the source layer's own weight may be stored too; it is not used (see ignored_tensors)
            tensors["value_mix.weight"] = TensorSpec(f"{p}.mix.vmix", (), init="unit_interval")
        mixer = PartSpec(
            "talking_heads_attention",
            {"dim": d, "n_heads": H, "n_kv_heads": G, "head_dim": hd, "value_dim": vd, "scale": float(m["scale"]),
             "window": mask.get("size"), "softcap": m.get("softcap"), "unit_norm_eps": eps, "distance_slopes": distance_slopes(H),
             "value_mix": value_mix, "value_mix_key": "first"},
            tensors, family="mixer")
        parts = {"norm1": rms_norm(f"{p}.norm1"), "mixer": mixer}
        mlp = layer.get("mlp")
        if mlp is not None:
            f = mlp["ff"]
            parts["feed_forward"] = PartSpec(
                "poly_norm_mlp", {"dim": d, "inner_dim": f, "eps": eps},
                {"up.weight": TensorSpec(f"{p}.mlp.up", (f, d), std=lin), "down.weight": TensorSpec(f"{p}.mlp.down", (d, f), std=1.0 / math.sqrt(f)),
                 "coefficients": TensorSpec(f"{p}.mlp.act", (4,), std=0.5)},
                family="feed_forward")
        parts["stream_mix"] = PartSpec("depth_weighted_average", {"index": i, "n_runs": n_layers},
                                       {"weights": TensorSpec(f"{p}.dwa", (i + 2,), init="last_one_plus_normal", std=0.2)}, family="stream_mix")
        layers.append(LayerSpec("parallel", parts))

    embedding = PartSpec("token_embedding", {"vocab_size": cfg.vocab, "dim": d, "position": None},
                         {"table": TensorSpec("embed", (cfg.vocab, d), std=1.0)}, family="embedding")
    head = PartSpec("tied_head", {"vocab_size": cfg.vocab, "dim": d}, {"table": TensorSpec("embed", (cfg.vocab, d), std=1.0)}, family="head")
    return ModelSpec(
        architecture="zederax",
        vocab_size=cfg.vocab,
        dim=d,
        embedding=embedding,
        layers=layers,
        plan=[PlanEntry(layer=i, cache=i, writes_cache=True) for i in range(n_layers)],
        final_norm=rms_norm("final.norm"),
        head=head,
        max_positions=None,
        # a blend weight that a file stores for a layer that does not blend (the values' source, a layer without the blend)
        ignored_tensors=(r"l\d+\.mix\.vmix",),
        init_std=cfg.initializer_range,
    )
