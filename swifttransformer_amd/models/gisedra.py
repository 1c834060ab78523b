"""Gisedra: a decoder of "sandwich" layers (a dynamic-tanh norm before and after each sublayer) whose
mixers are latent attention with a window and a shared rotated key part, or grouped window attention
beside a retention; feed-forwards of routed experts with softmax weights over the chosen; a gated
per-layer token embedding added at unit root mean square; and a group of layers that may run several
times in a row, each pass starting from the stream plus the embedding plus a vector of its own.

This module turns its config.json into a ``ModelSpec`` (which parts, which sizes, which tensor names) and
registers it; the parts themselves know nothing of it.  Tensor names of the folder's safetensors file:
``embed``, ``loop.step``, ``side.embed``, ``final.norm[.b|.alpha]``, ``head``, and per layer i
``l<i>.norm1|norm1b|norm2|norm2b[.b|.alpha]``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``l<i>.side.*``."""
from __future__ import annotations

from ..config.gisedra_param import ARCHITECTURE, GisedraHyperParam
from ..config.registry import register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry


def _norm(name: str) -> PartSpec:
    # tanh(alpha x) * w + b
    return PartSpec("dynamic_tanh", {}, {"weight": name, "bias": name + ".b", "alpha": name + ".alpha"})


def _latent(hp: GisedraHyperParam, p: str, mx: dict) -> PartSpec:
    rot = mx.get("rot") or {}
    return PartSpec("latent_attention",
                    {"num_heads": mx["heads"], "key_dim": mx["dim"], "value_dim": mx["vdim"], "rank": mx["kv_rank"],
                     "scale": float(mx["scale"]), "eps": hp.norm_eps, "rot_dim": mx["rot_dim"],
                     "rot_dims": int(rot.get("dims", mx["rot_dim"]) or 0), "rot_base": float(rot.get("base", 10000.0)),
                     "rot_scaling": rot.get("scaling"),
                     "window": int((mx.get("mask") or {}).get("size", 0))},
                    {"q": f"{p}.q", "down": f"{p}.dkv", "down_norm": f"{p}.dkv.norm", "up_k": f"{p}.uk",
                     "up_v": f"{p}.uv", "out": f"{p}.o"})


def _parallel(hp: GisedraHyperParam, p: str, mx: dict) -> PartSpec:
    left, right = mx["left"], mx["right"]
    rot, mask = left.get("rot"), left.get("mask") or {}
    rotary = None
    if rot is not None:
        rotary = PartSpec("rotary", {"head_dim": left["dim"], "dims": rot["dims"], "base": float(rot["base"]),
                                     "scaling": rot.get("scaling")})
    lp, rp = f"{p}.left", f"{p}.right"
    left_spec = PartSpec("gated_window_attention",
                         {"num_heads": left["heads"], "num_kv_heads": left["kv_heads"], "key_dim": left["dim"],
                          "value_dim": left["vdim"], "scale": float(left["scale"]), "window": int(mask.get("size", 0)),
                          "keep_first": int(mask.get("keep_first", 0) or 0), "taps": int(left.get("conv") or 0),
                          "rotary": rotary, "gate": "sigmoid", "out_scale": float(mx["left_scale"])},
                         {"q": f"{lp}.q", "k": f"{lp}.k", "v": f"{lp}.v", "gate": f"{lp}.g", "out": f"{lp}.o",
                          "q_conv": f"{lp}.q.conv", "k_conv": f"{lp}.k.conv", "v_conv": f"{lp}.v.conv"})
    right_spec = PartSpec("retention",
                          {"num_heads": right["heads"], "key_dim": right["dim"], "value_dim": right["vdim"],
                           "decay": list(right["decay"]), "eps": hp.norm_eps, "out_scale": float(mx["right_scale"])},
                          {"q": f"{rp}.q", "k": f"{rp}.k", "v": f"{rp}.v", "gate": f"{rp}.g", "out": f"{rp}.o"})
    return PartSpec("parallel", {"left": left_spec, "right": right_spec})


def build_gisedra_spec(hp: GisedraHyperParam) -> ModelSpec:
    hp.validate()
    layers = []
    n = len(hp.layers)
    for i, L in enumerate(hp.layers):
        p, mlp = f"l{i}", L.get("mlp")
        mixer = (_latent(hp, f"{p}.mix", L["mixer"]) if L["type"] == "latent_attention"
                 else _parallel(hp, f"{p}.mix", L["mixer"]))
        ffn = None
        if mlp is not None:
            ffn = PartSpec("routed_experts",
                           {"experts": mlp["router"]["experts"], "top": mlp["router"]["top"], "inner": mlp["expert"]["ff"],
                            "style": "softmax_output", "router_bias": True},
                           {"router": f"{p}.mlp.router", "router_bias": f"{p}.mlp.router.b",
                            "gate": p + ".mlp.e{e}.gate", "up": p + ".mlp.e{e}.up", "down": p + ".mlp.e{e}.down"})
        side = None
        if hp.token_side_dim:
            side = PartSpec("token_side", {"vocab_size": hp.vocab, "dim": hp.token_side_dim, "index": i, "parts": n,
                                           "eps": hp.norm_eps},
                            {"table": "side.embed", "gate": f"{p}.side.gate", "proj": f"{p}.side.proj",
                             "norm": f"{p}.side.norm"})
        layers.append(LayerSpec(
            arrangement=PartSpec("sandwich", {"feed_forward": ffn is not None}),
            mixer_norm=_norm(f"{p}.norm1"), mixer=mixer, mixer_out_norm=_norm(f"{p}.norm1b"),
            ffn_norm=_norm(f"{p}.norm2") if ffn is not None else None, feed_forward=ffn,
            ffn_out_norm=_norm(f"{p}.norm2b") if ffn is not None else None, side_input=side))
    # every run of a layer has caches and states of its own; the first layer of each pass over the repeated
    # group is entered through that pass's sum of the stream, the embedding (from the second pass on) and
    # the pass's vector
    entries, schedule = [], []
    times = int(hp.loop["times"]) if hp.loop is not None else 0
    for run, (i, pass_no) in enumerate(hp.run_order()):
        enter = None
        if pass_no is not None:
            enter = len(entries)
            entries.append(PartSpec("additive", {"index": pass_no, "passes": times, "add_first": pass_no > 0},
                                    {"shift": "loop.step"}))
        schedule.append(ScheduleEntry(layer=i, cache=run, enter=enter))
    return ModelSpec(
        hidden_size=hp.width, vocab_size=hp.vocab, max_positions=hp.max_positions,
        embedding=PartSpec("token", {"vocab_size": hp.vocab, "embed_dim": hp.width}, {"weight": "embed"}),
        position=PartSpec("none"),
        layers=layers, schedule=schedule, entries=entries,
        final_norm=_norm("final.norm"),
        head=PartSpec("linear", {"vocab_size": hp.vocab, "embed_dim": hp.width, "tied_to": None}, {"weight": "head"}),
        eos_token_id=hp.eos_token_id,
    ).validate()


def _presets(name: str, **overrides) -> GisedraHyperParam:
    from ..config.presets import gisedra_preset
    return gisedra_preset(name, **overrides)


register_architecture(ARCHITECTURE, GisedraHyperParam, build_gisedra_spec, short_name="gisedra", presets=_presets)
