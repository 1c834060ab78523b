"""Pupalix: a decoder of pre-norm layers whose mixers are latent attention with a shared rotated key part,
grouped attention whose values are its keys (capped scores, a mask of chunks), or lightning attention; dense
gated or group-routed expert feed-forwards; a token embedding with a hashed pair table; a residual stream of
several copies with learned reads and writes; a group of layers that may run several times; a tied head with a
factor and a smooth limit on the logits.

This module turns its config.json into a ``ModelSpec`` and registers it; the parts themselves know nothing
of it.  Tensor names of the folder's safetensors file: ``embed``, ``bigram``, ``final.norm`` and per layer i
``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.hc1|hc2.in|out|mix``."""
from __future__ import annotations

from ..config.pupalix_param import ARCHITECTURE, PupalixHyperParam
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def _norm(hp: PupalixHyperParam, name: str) -> PartSpec:
    return PartSpec("layer_norm", {"eps": hp.norm_eps, "center": False, "bias": False}, {"weight": name})


def _mixer(hp: PupalixHyperParam, kind: str, p: str, mx: dict) -> PartSpec:
    if kind == "latent_attention":
        rot = mx.get("rot") or {}
        return PartSpec("latent_attention",
                        {"num_heads": mx["heads"], "key_dim": mx["dim"], "value_dim": mx["vdim"], "rank": mx["kv_rank"],
                         "scale": float(mx["scale"]), "eps": hp.norm_eps, "rot_dim": mx["rot_dim"],
                         "rot_dims": int(rot.get("dims", mx["rot_dim"]) or 0), "rot_base": float(rot.get("base", 10000.0)),
                         "rot_scaling": rot.get("scaling"), "window": 0},
                        {"q": f"{p}.q", "down": f"{p}.dkv", "down_norm": f"{p}.dkv.norm", "up_k": f"{p}.uk",
                         "up_v": f"{p}.uv", "out": f"{p}.o"})
    if kind == "attention":
        return PartSpec("tied_kv_attention",
                        {"num_heads": mx["heads"], "num_kv_heads": mx["kv_heads"], "head_dim": mx["dim"],
                         "scale": float(mx["scale"]), "eps": hp.norm_eps, "softcap": float(mx.get("softcap") or 0.0),
                         "chunk": int((mx.get("mask") or {}).get("size", 0))},
                        {"q": f"{p}.q", "k": f"{p}.k", "q_norm": f"{p}.q.norm", "k_norm": f"{p}.k.norm", "out": f"{p}.o"})
    return PartSpec("retention",
                    {"num_heads": mx["heads"], "key_dim": mx["dim"], "value_dim": mx["vdim"], "decay": list(mx["decay"]),
                     "eps": hp.norm_eps, "qkv_activation": "silu", "key_scale": 1.0, "norm": "all", "gate": "sigmoid"},
                    {"q": f"{p}.q", "k": f"{p}.k", "v": f"{p}.v", "gate": f"{p}.g", "out": f"{p}.o", "norm": f"{p}.norm"})


def _feed_forward(p: str, mlp):
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return PartSpec("gated_dense", {"inner": mlp["ff"], "activation": "gelu_tanh"},
                        {"gate": f"{p}.gate", "up": f"{p}.up", "down": f"{p}.down"})
    r = mlp["router"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    return PartSpec("routed_experts",
                    {"experts": r["experts"], "top": r["top"], "inner": mlp["expert"]["ff"], "style": "softmax_all",
                     "groups": g["count"], "keep": g["keep"]},
                    {"router": f"{p}.router", "gate": p + ".e{e}.gate", "up": p + ".e{e}.up", "down": p + ".e{e}.down"})


def build_pupalix_spec(hp: PupalixHyperParam) -> ModelSpec:
    hp.validate()
    layers = []
    for i, L in enumerate(hp.layers):
        p = f"l{i}"
        ffn = _feed_forward(f"{p}.mlp", L.get("mlp"))
        if hp.streams:
            names = {f"{side}_{what}": f"{p}.{hc}.{what}" for side, hc in (("mixer", "hc1"), ("ffn", "hc2"))
                     for what in ("in", "out", "mix")}
            if ffn is None:
                names["unused_norm"] = f"{p}.norm2"
            arrangement = PartSpec("hyper_connections", {"streams": hp.streams, "feed_forward": ffn is not None}, names)
        else:
            arrangement = PartSpec("pre_norm", {"feed_forward": ffn is not None})
        layers.append(LayerSpec(
            arrangement=arrangement, mixer_norm=_norm(hp, f"{p}.norm1"),
            mixer=_mixer(hp, L["type"], f"{p}.mix", L["mixer"]),
            ffn_norm=_norm(hp, f"{p}.norm2") if ffn is not None else None, feed_forward=ffn))
    # every run of a layer has a cache or state of its own
    schedule = [ScheduleEntry(layer=i, cache=run) for run, i in enumerate(hp.run_order())]
    if hp.bigram is not None:
        embedding = PartSpec("hashed_pairs", {"vocab_size": hp.vocab, "scale": hp.embedding_scale, **hp.bigram},
                             {"weight": "embed", "pairs": "bigram"})
    else:
        embedding = PartSpec("hashed_pairs", {"vocab_size": hp.vocab, "scale": hp.embedding_scale, "buckets": 0},
                             {"weight": "embed"})
    return ModelSpec(
        hidden_size=hp.width, vocab_size=hp.vocab, max_positions=hp.max_positions,
        embedding=embedding, position=PartSpec("none"),
        layers=layers, schedule=schedule, streams=hp.streams,
        final_norm=_norm(hp, "final.norm"),
        head=PartSpec("linear", {"vocab_size": hp.vocab, "embed_dim": hp.width, "tied_to": "embed",
                                 "logit_scale": hp.logit_scale, "softcap": hp.logit_softcap}, {"weight": "head"}),
        eos_token_id=hp.eos_token_id,
    ).validate()


def _presets(name: str, **overrides) -> PupalixHyperParam:
    from ..config.presets import pupalix_preset
    return pupalix_preset(name, **overrides)


register_architecture(ARCHITECTURE, PupalixHyperParam, build_pupalix_spec, short_name="pupalix", presets=_presets)
