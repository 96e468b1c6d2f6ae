"""Pafivik: a decoder whose layers choose among three mixers, with a norm on both sides of every sublayer and an
average over depth behind every layer.

config.json: `vocab`, `width`, `norm.eps`, `embedding.scale`, `residual_mult`, `layers` (each: `type`, `mixer` with the
mixer's sizes and constants, `mlp` or null).  Optional: `max_positions` (the engine's limit on a request's length; the
architecture itself has none).  The inner sizes of a channel_delta mixer's two pairs of small matrices are not in
config.json: the tensors give them by their shape (`with_shapes`), and weights made here take `decay_rank` / `gate_rank`
from the mixer's entry if it names them.

The model: x = embed[token] * embedding.scale.  Layer i: x += m * ls1 * norm1b(mixer(norm1(x))), then, if it has a
feed-forward, x += m * ls2 * norm2b(ff(norm2(x))), with m = residual_mult, all four norms root-mean-square norms with a
weight, ls1 and ls2 vectors of the layer.  With X_0 the embedded rows and X_(i+1) what layer i leaves, what goes on to the
next layer (and, behind the last, to the final norm) is sum_j dwa_i[j] X_j over j = 0 .. i + 1.  The head is the token
table itself, without the embedding's scale.

Mixers: "lightning" and "channel_delta" (parts.recurrent), "attention" (parts.mixers.CausalSelfAttention with biases,
grouped key heads, values of a width of their own, pairs of the first rot.dims dimensions turned by the position, the
score's scale from config.json).  Feed-forwards: "dense" (parts.feedforward.DenseMLP with the xielu activation and
biases) and "moe" (parts.feedforward.RoutedExperts: sigmoid scores, the chosen scores as weights, the weight on what the
expert reads, silu-gated experts without biases, a shared expert behind a gate per token).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass

from ..config.base import ConfigError, read_float, read_int, read_str
from ..config.registry import register_architecture
from ..parts.model import DecoderSpec, LayerCall, LayerSpec

MIXER_TYPES = ("lightning", "channel_delta", "attention")
DEFAULT_MAX_POSITIONS = 65536
DEFAULT_RANK = 16        # for weights made here; a checkpoint's own tensors say theirs


def _sub(d, key, where="config.json"):
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: key '{key}' must be an object")
    return v


@dataclass(frozen=True)
class PafivikConfig:
    raw: dict

    architecture = "Pafivik"

    @property
    def vocab(self):
        return self.raw["vocab"]

    @property
    def width(self):
        return self.raw["width"]

    @property
    def eps(self):
        return float(self.raw["norm"]["eps"])

    @property
    def layers(self):
        return self.raw["layers"]

    @property
    def max_positions(self):
        return self.raw.get("max_positions") or DEFAULT_MAX_POSITIONS

    @classmethod
    def from_dict(cls, d: dict) -> "PafivikConfig":
        raw = copy.deepcopy({k: v for k, v in d.items() if k not in ("architectures", "torch_dtype")})
        read_int(raw, "vocab", minimum=1), read_int(raw, "width", minimum=1)
        read_float(_sub(raw, "norm"), "eps")
        read_float(_sub(raw, "embedding"), "scale")
        read_float(raw, "residual_mult")
        read_int(raw, "max_positions", default=None, minimum=1)
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: key 'layers' must be a list of layers")
        for i, layer in enumerate(layers):
            where = f"config.json: layers[{i}]"
            if not isinstance(layer, dict):
                raise ConfigError(f"{where} must be an object")
            kind = read_str(layer, "type", choices=MIXER_TYPES)
            m = _sub(layer, "mixer", where)
            heads = read_int(m, "heads", minimum=1)
            read_int(m, "dim", minimum=1), read_int(m, "vdim", minimum=1)
            if kind == "lightning":
                decay = m.get("decay")
                if not isinstance(decay, list) or len(decay) != heads or not all(isinstance(x, (int, float)) for x in decay):
                    raise ConfigError(f"{where}.mixer.decay must be a list of {heads} numbers, one per head")
            else:
                kv = read_int(m, "kv_heads", minimum=1)
                if heads % kv != 0:
                    raise ConfigError(f"{where}.mixer: heads ({heads}) is no multiple of kv_heads ({kv})")
            if kind == "channel_delta":
                read_int(m, "conv", minimum=1)
                read_int(m, "decay_rank", default=None, minimum=1), read_int(m, "gate_rank", default=None, minimum=1)
            if kind == "attention":
                read_float(m, "scale")
                if m.get("rot") is not None:
                    rot = _sub(m, "rot", where + ".mixer")
                    read_float(rot, "base")
                    dims = read_int(rot, "dims", minimum=0)
                    if dims % 2 or dims > m["dim"]:
                        raise ConfigError(f"{where}.mixer.rot.dims = {dims}: an even number up to dim ({m['dim']})")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict):
                    raise ConfigError(f"{where}.mlp must be an object or null")
                if read_str(mlp, "kind", choices=("dense", "moe")) == "dense":
                    read_int(mlp, "ff", minimum=1)
                else:
                    read_int(_sub(mlp, "expert", where + ".mlp"), "ff", minimum=1)
                    ro = _sub(mlp, "router", where + ".mlp")
                    n, top = read_int(ro, "experts", minimum=1), read_int(ro, "top", minimum=1)
                    if top > n:
                        raise ConfigError(f"{where}.mlp.router: top ({top}) is more than experts ({n})")
                    if mlp.get("shared") is not None:
                        read_int(_sub(mlp, "shared", where + ".mlp"), "ff", minimum=1)
        return cls(raw)

    def with_shapes(self, shapes: dict) -> "PafivikConfig":
        """Sizes that config.json leaves to the tensors: the inner sizes of a channel_delta mixer's small matrices are
        the row counts of the first of each pair."""
        raw = copy.deepcopy(self.raw)
        for i, layer in enumerate(raw["layers"]):
            if layer["type"] != "channel_delta":
                continue
            for key, name in (("decay_rank", "a1"), ("gate_rank", "g1")):
                shape = shapes.get(f"l{i}.mix.{name}")
                if shape is not None and len(shape) == 2:
                    layer["mixer"][key] = int(shape[0])
        return PafivikConfig(raw)

    def to_dict(self) -> dict:
        d = copy.deepcopy(self.raw)
        d["architecture"] = self.architecture
        return d


def _mixer(cfg: PafivikConfig, i: int, layer: dict):
    m, p, W = layer["mixer"], f"l{i}.mix.", cfg.width
    if layer["type"] == "lightning":
        return ("lightning", dict(width=W, n_heads=m["heads"], head_dim=m["dim"], value_dim=m["vdim"], decay=m["decay"], eps=cfg.eps,
                                  names={s: p + s for s in ("q", "k", "v", "g", "o", "norm")}))
    if layer["type"] == "channel_delta":
        names = {s: p + s for s in ("q", "k", "v", "b", "a1", "a2", "g1", "g2", "o", "A_log", "dt_bias", "norm")}
        names.update({s + "_conv": p + s + ".conv" for s in "qkv"})
        return ("channel_delta", dict(width=W, n_heads=m["heads"], n_qk_heads=m["kv_heads"], head_dim=m["dim"], value_dim=m["vdim"],
                                      taps=m["conv"], eps=cfg.eps, decay_rank=m.get("decay_rank") or DEFAULT_RANK,
                                      gate_rank=m.get("gate_rank") or DEFAULT_RANK, names=names))
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot")
    return ("causal_attention", dict(
        width=W, n_heads=H, n_kv_heads=G, head_dim=dk, value_dim=dv, scale=m["scale"], exact_turn=True,
        qkv_weight=p + "q+k+v", qkv_bias=p + "q+k+v.b", out_weight=p + "o", out_bias=None,
        qkv_weight_sources=((p + "q", H * dk), (p + "k", G * dk), (p + "v", G * dv)),
        qkv_bias_sources=((p + "q.b", H * dk), (p + "k.b", G * dk), (p + "v.b", G * dv)),
        position=("rotary_pairs", dict(dims=rot["dims"], base=rot["base"], head_dim=dk)) if rot else None))


def _feed_forward(cfg: PafivikConfig, i: int, mlp):
    p, W = f"l{i}.mlp.", cfg.width
    if mlp is None:
        return ("none", {})
    if mlp["kind"] == "dense":
        return ("dense_mlp", dict(width=W, inner=mlp["ff"], activation="xielu", activation_params=p + "act", up_weight=p + "up",
                                  up_bias=p + "up.b", down_weight=p + "down", down_bias=p + "down.b"))
    sh = mlp.get("shared")
    shared = dict(inner=sh["ff"], gate=p + "shared.gate", up=p + "shared.up", down=p + "shared.down",
                  token_gate=p + "shared.sg") if sh else None
    return ("routed_experts", dict(
        width=W, inner=mlp["expert"]["ff"], n_experts=mlp["router"]["experts"], top=mlp["router"]["top"], router=p + "router",
        correction=None, gate=p + "e{e}.gate", up=p + "e{e}.up", down=p + "e{e}.down", score="sigmoid", renorm=False,
        weigh="input", act="silu", shared=shared))


def build_pafivik(cfg: PafivikConfig) -> DecoderSpec:
    W, mult = cfg.width, float(cfg.raw["residual_mult"])

    def norm(name):
        return ("rmsnorm", dict(width=W, eps=cfg.eps, weight_name=name))

    def post(name, scale):
        return ("rmsnorm_into_stream", dict(width=W, eps=cfg.eps, weight_name=name, scale_name=scale, mult=mult))
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        layers.append(LayerSpec(arrangement="sandwich", parts=dict(
            norm1=norm(p + "norm1"), mixer=_mixer(cfg, i, layer), post1=post(p + "norm1b", p + "ls1"),
            norm2=norm(p + "norm2"), ffn=_feed_forward(cfg, i, layer.get("mlp")), post2=post(p + "norm2b", p + "ls2"))))
    order = [LayerCall(layer=i, cache=i, average=f"l{i}.dwa") for i in range(len(cfg.layers))]
    return DecoderSpec(
        vocab=cfg.vocab, width=W, max_positions=cfg.max_positions, token_table="embed", position=("none", {}),
        layers=layers, run_order=order, final_norm=norm("final.norm"), head_weight=None,
        embedding_scale=float(cfg.raw["embedding"]["scale"]),
        # (a layer without a feed-forward has no use for its second pair of norms, whether or not a file holds them)
        ignore_tensors=tuple(rf"^l{i}\.(norm2|norm2b|ls2)$" for i, layer in enumerate(cfg.layers) if layer.get("mlp") is None))


register_architecture(["Pafivik"], PafivikConfig, build_pafivik)
