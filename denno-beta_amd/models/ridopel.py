"""Ridopel: a decoder whose layers take turns between three mixers, with a loop over a run of layers.

config.json: `vocab`, `width`, `norm.eps`, `canon.taps` (absent: no input convolution), `logit_softcap` (absent: none),
`layers` (each: `type`, `mixer` with the mixer's sizes, `mlp` or null) and `loop` (`start`, `stop`, `times`; absent: every
layer runs once).  Optional: `max_positions` (the engine's limit on a request's length; the architecture itself has
none) and, in a wkv mixer, `decay_rank` (the inner size of the decay's two small matrices, which a checkpoint's tensors
give by their shape) and, in a latent_attention mixer, `keep` ("latent" or "heads": what the cache holds, see
parts.mixers.LatentAttention; absent: the latent where the attention kernels take its width).

The model: token rows, normed; then the layers in their order, layers start .. stop - 1 `times` times in a row with the
same weights and a cache of their own per pass; before the first layer of every pass the stream becomes
W_in [x ; x0] with x0 the normed token rows.  A layer: x += mixer(conv(norm1(x))), then x += experts(norm2(x)) if it has
a feed-forward.  All norms are root-mean-square norms with a weight.  Then the final norm, the head, and a soft cap.

Mixers: "latent_attention" (parts.mixers.LatentAttention), "wkv" and "hgrn2" (parts.recurrent); feed-forward:
a mixture of experts (parts.feedforward.RoutedExperts) whose activation constant 1.702 the architecture fixes.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Optional

from ..config.base import ConfigError, read_float, read_int, read_str
from ..config.registry import register_architecture
from ..parts.model import DecoderSpec, LayerCall, LayerSpec

MIXER_TYPES = ("latent_attention", "wkv", "hgrn2")
EXPERT_ALPHA = 1.702
DEFAULT_MAX_POSITIONS = 65536
DEFAULT_DECAY_RANK = 32        # for weights made here; a checkpoint's own tensors say theirs


def _sub(d, key, where="config.json"):
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: key '{key}' must be an object")
    return v


@dataclass(frozen=True)
class RidopelConfig:
    raw: dict

    architecture = "Ridopel"

    # -- typed access ------------------------------------------------------------------------------
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
    def taps(self):
        return self.raw["canon"]["taps"] if self.raw.get("canon") else 0

    @property
    def layers(self):
        return self.raw["layers"]

    @property
    def max_positions(self):
        return self.raw.get("max_positions") or DEFAULT_MAX_POSITIONS

    def run_order(self):
        """[(layer, whether a pass of the loop starts here)] in the order in which layers run."""
        n, loop = len(self.layers), self.raw.get("loop")
        if not loop:
            return [(i, False) for i in range(n)]
        a, b, times = loop["start"], loop["stop"], loop["times"]
        order = [(i, False) for i in range(a)]
        for _ in range(times):
            order += [(i, i == a) for i in range(a, b)]
        return order + [(i, False) for i in range(b, n)]

    # -- reading -----------------------------------------------------------------------------------
    @classmethod
    def from_dict(cls, d: dict) -> "RidopelConfig":
        raw = copy.deepcopy({k: v for k, v in d.items() if k not in ("architectures", "torch_dtype")})
        read_int(raw, "vocab", minimum=1), read_int(raw, "width", minimum=1)
        read_float(_sub(raw, "norm"), "eps")
        if raw.get("canon") is not None:
            read_int(_sub(raw, "canon"), "taps", minimum=1)
        if raw.get("logit_softcap") is not None:
            read_float(raw, "logit_softcap")
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
            read_int(m, "heads", minimum=1), read_int(m, "dim", minimum=1)
            if kind == "latent_attention":
                for key in ("kv_rank", "rot_dim", "vdim"):
                    read_int(m, key, minimum=1)
                read_float(m, "scale")
                rot = _sub(m, "rot", where + ".mixer")
                read_float(rot, "base")
                dims = read_int(rot, "dims", minimum=0)
                if dims % 2 or dims > m["rot_dim"]:
                    raise ConfigError(f"{where}.mixer.rot.dims = {dims}: an even number up to rot_dim ({m['rot_dim']})")
            elif kind == "hgrn2":
                read_int(m, "vdim", minimum=1)
            else:
                read_int(m, "decay_rank", default=None, minimum=1)
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict):
                    raise ConfigError(f"{where}.mlp must be an object or null")
                read_str(mlp, "kind", choices=("moe",))
                ex, ro = _sub(mlp, "expert", where + ".mlp"), _sub(mlp, "router", where + ".mlp")
                read_int(ex, "ff", minimum=1), read_float(ex, "limit")
                n, top = read_int(ro, "experts", minimum=1), read_int(ro, "top", minimum=1)
                if top > n:
                    raise ConfigError(f"{where}.mlp.router: top ({top}) is more than experts ({n})")
        loop = raw.get("loop")
        if loop is not None:
            if not isinstance(loop, dict):
                raise ConfigError("config.json: key 'loop' must be an object")
            a, b = read_int(loop, "start", minimum=0), read_int(loop, "stop", minimum=0)
            read_int(loop, "times", minimum=1)
            if not a < b <= len(layers):
                raise ConfigError(f"config.json: loop.start ({a}) < loop.stop ({b}) <= {len(layers)} layers does not hold")
        return cls(raw)

    def with_shapes(self, shapes: dict) -> "RidopelConfig":
        """Sizes that config.json leaves to the tensors: a wkv mixer's decay rank is the first matrix's row count."""
        raw = copy.deepcopy(self.raw)
        for i, layer in enumerate(raw["layers"]):
            shape = shapes.get(f"l{i}.mix.w1")
            if layer["type"] == "wkv" and shape is not None and len(shape) == 2:
                layer["mixer"]["decay_rank"] = int(shape[0])
        return RidopelConfig(raw)

    def to_dict(self) -> dict:
        d = copy.deepcopy(self.raw)
        d["architecture"] = self.architecture
        return d


def _mixer(cfg: RidopelConfig, i: int, layer: dict):
    m, p, W = layer["mixer"], f"l{i}.mix.", cfg.width
    if layer["type"] == "latent_attention":
        return ("latent_attention", dict(
            width=W, n_heads=m["heads"], head_dim=m["dim"], rot_dim=m["rot_dim"], value_dim=m["vdim"], kv_rank=m["kv_rank"],
            scale=m["scale"], eps=cfg.eps, position=dict(dims=m["rot"]["dims"], base=m["rot"]["base"]), keep=m.get("keep"),
            names=dict(q=p + "q", dkv=p + "dkv", g=p + "g", uk=p + "uk", uv=p + "uv", o=p + "o", dkv_norm=p + "dkv.norm")))
    if layer["type"] == "wkv":
        names = {s: p + s for s in ("r", "k", "v", "g", "w1", "w2", "o", "w0", "u", "norm")}
        names.update({"mu_" + s: p + "mu." + s for s in "rkvgw"})
        return ("wkv", dict(width=W, n_heads=m["heads"], head_dim=m["dim"], eps=cfg.eps,
                            lora=m.get("decay_rank") or DEFAULT_DECAY_RANK, names=names))
    return ("hgrn2", dict(width=W, n_heads=m["heads"], head_dim=m["dim"], value_dim=m["vdim"], eps=cfg.eps,
                          names=dict(q=p + "q", f=p + "f", v=p + "v", o=p + "o", f_bias=p + "f.b", lower=p + "lower",
                                     norm=p + "norm")))


def build_ridopel(cfg: RidopelConfig) -> DecoderSpec:
    W = cfg.width

    def norm(name):
        return ("rmsnorm", dict(width=W, eps=cfg.eps, weight_name=name))
    layers = []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        mlp = layer.get("mlp")
        ffn = ("none", {}) if mlp is None else ("routed_experts", dict(
            width=W, inner=mlp["expert"]["ff"], n_experts=mlp["router"]["experts"], top=mlp["router"]["top"],
            limit=mlp["expert"]["limit"], alpha=EXPERT_ALPHA, router=p + "mlp.router", correction=p + "mlp.correction",
            gate=p + "mlp.e{e}.gate", up=p + "mlp.e{e}.up", down=p + "mlp.e{e}.down"))
        conv = ("causal_conv", dict(width=W, taps=cfg.taps, weight_name=p + "canon1")) if cfg.taps else ("none", {})
        layers.append(LayerSpec(arrangement="pre_norm_filtered", parts=dict(
            norm1=norm(p + "norm1"), filter=conv, mixer=_mixer(cfg, i, layer), norm2=norm(p + "norm2"), ffn=ffn)))
    # every run of a layer has caches of its own: one for the input convolution's history, one for the mixer
    order = [LayerCall(layer=i, cache=(2 * n, 2 * n + 1), inject="loop" if first else None)
             for n, (i, first) in enumerate(cfg.run_order())]
    return DecoderSpec(
        vocab=cfg.vocab, width=W, max_positions=cfg.max_positions, token_table="embed", position=("none", {}),
        layers=layers, run_order=order, final_norm=norm("final.norm"), head_weight="head",
        logit_softcap=float(cfg.raw.get("logit_softcap") or 0.0), embedding_norm=norm("embed.norm"),
        injections={"loop": "loop.in"} if cfg.raw.get("loop") else {},
        # (a layer without a feed-forward has no use for a second norm, whether or not a file holds one)
        ignore_tensors=tuple(rf"^l{i}\.norm2$" for i, layer in enumerate(cfg.layers) if layer.get("mlp") is None))


register_architecture(["Ridopel"], RidopelConfig, build_ridopel)
