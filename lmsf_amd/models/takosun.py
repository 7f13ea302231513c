"""Takosun as a ModelSpec: a decoder whose layers attend over a cached latent.

Every layer: a norm in groups before and after each sublayer, attention over a latent that the layer caches
itself or reads from an earlier layer's cache (``kv_from``), a dense gated feed-forward or experts assigned by
a table of token ids with a shared expert (or no feed-forward), and a learned weighted average over the results
of all layers so far. The reference has no such architecture; its model files hard-wire Llama's block
(core/src/model_executor/models/llama/llama.rs:276-385).

config.json: "architecture": "Takosun", "vocab", "width", "norm": {"eps", "groups"}, and "layers", a list of
{"type": "latent_attention", "mixer": {"heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "scale",
"rot": {"base", "dims"}, "kv_from"?}, "mlp": null | {"kind": "dense", "ff"} | {"kind": "moe", "expert": {"ff"},
"router": {"experts", "top"}, "shared": {"ff"}?}}. Optional: "max_position_embeddings", "torch_dtype",
"eos_token_id", "bos_token_id".

Checkpoint names: embed, head, final.norm; per layer l<i>.{norm1, norm1b, norm2, norm2b, dwa},
l<i>.mix.{dq, dq.norm, uq, dkv, dkv.norm, uk, uv, g, o}, l<i>.mlp.{gate, up, down} or
l<i>.mlp.{table, e<k>.{gate, up, down}, shared.{gate, up, down}}.
"""
import dataclasses
import json
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.model_config import ArchConfig, ConfigError
from ..config.registry import register_architecture
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

DEFAULT_MAX_POSITIONS = 131072


def _need(d: Dict[str, Any], key: str, where: str, kind=(int,), positive: bool = True):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError("config.json: %s lacks %r" % (where, key))
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, kind):
        raise ConfigError("config.json: %s.%s is %r" % (where, key, v))
    if positive and not v > 0:
        raise ConfigError("config.json: %s.%s must be > 0, is %r" % (where, key, v))
    return v


@dataclass(frozen=True)
class TakosunConfig(ArchConfig):
    width: int = 0
    norm_eps: float = 1e-5
    norm_groups: int = 1
    layers_json: str = "[]"        # the "layers" list as it was read (kept as text: the dataclass is frozen and hashable)

    ARCHITECTURE = "Takosun"

    @property
    def layers(self) -> Tuple[Dict[str, Any], ...]:
        return tuple(json.loads(self.layers_json))

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "TakosunConfig":
        vocab = _need(d, "vocab", "the configuration")
        width = _need(d, "width", "the configuration")
        norm = d.get("norm")
        eps = _need(norm, "eps", "norm", (int, float))
        groups = _need(norm, "groups", "norm")
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        cfg = cls(architecture=cls.ARCHITECTURE, vocab_size=int(vocab),
                  max_position_embeddings=int(d.get("max_position_embeddings") or DEFAULT_MAX_POSITIONS),
                  torch_dtype=str(d.get("torch_dtype") or "bfloat16"), eos_token_ids=eos_ids,
                  bos_token_id=None if d.get("bos_token_id") is None else int(d["bos_token_id"]),
                  width=int(width), norm_eps=float(eps), norm_groups=int(groups), layers_json=json.dumps(layers))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.width % self.norm_groups:
            raise ConfigError("config.json: width %d does not split into norm.groups %d" % (self.width, self.norm_groups))
        owners = {}
        for i, layer in enumerate(self.layers):
            where = "layers[%d]" % i
            if not isinstance(layer, dict) or layer.get("type") != "latent_attention":
                raise ConfigError("config.json: %s.type %r is not supported (latent_attention)"
                                  % (where, layer.get("type") if isinstance(layer, dict) else layer))
            m = layer.get("mixer")
            for key in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"):
                _need(m, key, where + ".mixer")
            _need(m, "scale", where + ".mixer", (int, float))
            rot = m.get("rot")
            _need(rot, "base", where + ".mixer.rot", (int, float))
            dims = _need(rot, "dims", where + ".mixer.rot")
            if dims % 2 or dims > m["rot_dim"]:
                raise ConfigError("config.json: %s.mixer.rot.dims %d must be even and at most rot_dim %d"
                                  % (where, dims, m["rot_dim"]))
            src = m.get("kv_from")
            if src is None:
                owners[i] = (m["kv_rank"], m["rot_dim"], rot["base"], dims)
            else:
                if isinstance(src, bool) or not isinstance(src, int) or src not in owners:
                    raise ConfigError("config.json: %s.mixer.kv_from %r names no earlier layer with a latent of its own"
                                      % (where, src))
                if owners[src] != (m["kv_rank"], m["rot_dim"], rot["base"], dims):
                    raise ConfigError("config.json: %s.mixer reads the latent of layer %d, whose sizes or rotation differ"
                                      % (where, src))
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            kind = mlp.get("kind") if isinstance(mlp, dict) else None
            if kind == "dense":
                _need(mlp, "ff", where + ".mlp")
            elif kind == "moe":
                _need(mlp.get("expert"), "ff", where + ".mlp.expert")
                e = _need(mlp.get("router"), "experts", where + ".mlp.router")
                top = _need(mlp.get("router"), "top", where + ".mlp.router")
                if top > e:
                    raise ConfigError("config.json: %s.mlp.router.top %d exceeds experts %d" % (where, top, e))
                if mlp.get("shared") is not None:
                    _need(mlp["shared"], "ff", where + ".mlp.shared")
            else:
                raise ConfigError("config.json: %s.mlp.kind %r is not supported (dense, moe)" % (where, kind))

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.ARCHITECTURE, "vocab": self.vocab_size, "width": self.width,
                "norm": {"eps": self.norm_eps, "groups": self.norm_groups}, "layers": list(self.layers),
                "max_position_embeddings": self.max_position_embeddings, "torch_dtype": self.torch_dtype,
                "eos_token_id": list(self.eos_token_ids) or None, "bos_token_id": self.bos_token_id}


def build_takosun_spec(cfg: TakosunConfig) -> ModelSpec:
    W, L = cfg.width, len(cfg.layers)

    def norm(name: str) -> PartSpec:
        return PartSpec("group_rms_norm", {"prefix": name, "size": W, "eps": cfg.norm_eps, "groups": cfg.norm_groups,
                                           "weight_name": ""})

    def gated(prefix: str, ff: int) -> PartSpec:
        return PartSpec("gated_mlp", {"prefix": prefix, "hidden_size": W, "intermediate_size": ff, "activation": "silu",
                                      "gate_name": "gate", "up_name": "up", "down_name": "down", "bare_names": True})

    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        m, mlp = layer["mixer"], layer.get("mlp")
        src: Optional[int] = m.get("kv_from")
        mixer = PartSpec("latent_attention", {
            "prefix": "mix", "hidden_size": W, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
            "v_head_dim": m["vdim"], "kv_rank": m["kv_rank"], "q_rank": m["q_rank"], "scale": m["scale"],
            "eps": cfg.norm_eps, "owns_latent": src is None,
            "position": PartSpec("rotary", {"head_dim": m["rot_dim"], "rotary_dim": m["rot"]["dims"],
                                            "theta": m["rot"]["base"], "style": "neox"})})
        norms = {"pre_mixer": norm("norm1"), "post_mixer": norm("norm1b")}
        if mlp is None:
            ffn = PartSpec("none", {})
        else:
            norms.update({"pre_ffn": norm("norm2"), "post_ffn": norm("norm2b")})
            if mlp["kind"] == "dense":
                ffn = gated("mlp", mlp["ff"])
            else:
                shared = mlp.get("shared")
                ffn = PartSpec("table_moe", {
                    "prefix": "mlp", "hidden_size": W, "expert_size": mlp["expert"]["ff"],
                    "num_experts": mlp["router"]["experts"], "top": mlp["router"]["top"], "vocab_size": cfg.vocab_size,
                    "shared": gated("shared", shared["ff"]) if shared is not None else None})
        block = PartSpec("sandwich_depth_average", {"depth": i + 1, "depth_total": L,
                                                    "mix": PartSpec("depth_mix", {"count": i + 2, "weight_name": "dwa"})})
        layers.append(LayerSpec(prefix="l%d" % i, block=block, mixer=mixer, feed_forward=ffn, norms=norms))
        schedule.append(ScheduleEntry(i, cache_from=src))
    return ModelSpec(
        embedding=PartSpec("token_embedding", {"prefix": "embed", "vocab_size": cfg.vocab_size, "hidden_size": W,
                                               "weight_name": ""}),
        layers=tuple(layers), schedule=tuple(schedule), final_norm=norm("final.norm"),
        head=PartSpec("lm_head", {"prefix": "head", "vocab_size": cfg.vocab_size, "hidden_size": W,
                                  "weight_name": "head"}),
        vocab_size=cfg.vocab_size, hidden_size=W)


# a layer without a feed-forward may still carry the norms of one
TAKOSUN_TOLERATED = (".norm2", ".norm2b")

register_architecture("Takosun", "takosun", TakosunConfig, build_takosun_spec, tolerated_tensors=TAKOSUN_TOLERATED)
