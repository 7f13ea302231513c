"""Niresun as a ModelSpec: a pre-norm decoder whose layers mix tokens in three ways.

Every layer is x += mixer(dyt(x)), then, where it has a feed-forward, x += ffn(dyt(x)), with Dynamic Tanh
(tanh(alpha x) w + b) in the place of a norm. The mixer is one of
- "mamba1": the selective scan (parts/recurrent.py: ``selective_scan``);
- "attention": softmax attention with biases, rotary positions over part of a head with Llama-3.1 frequency
  scaling, a mask by chunks of positions and an output gate (parts/flex_attention.py);
- "parallel": two mixers side by side on the same input, each output RMS-normed over the width, the mean of the
  two (parts/parallel.py): "left" causal attention behind short convolutions with unit-norm queries and keys and
  a query temperature, "right" the matrix memory of xLSTM (``matrix_memory``).
The feed-forward is dense and gated with the tanh form of GELU. The reference has no such architecture; its
model files hard-wire Llama's block (core/src/model_executor/models/llama/llama.rs:276-385).

config.json: "architecture": "Niresun", "vocab", "width", "norm": {"eps"}, and "layers", a list of
{"type": "mamba1" | "attention" | "parallel", "mixer": {...}, "mlp": null | {"kind": "dense", "ff"}} with
  mamba1:    {"inner", "state", "dt_rank", "conv"}
  attention: {"heads", "kv_heads", "dim", "vdim", "scale", "rot": {"base", "dims", "scaling"?: {"factor", "low",
              "high", "original"}}?, "mask": {"size"}?}
  parallel:  {"left": {"heads", "kv_heads", "dim", "vdim", "scale", "conv", "q_temp": {"coef", "every"}?},
              "right": {"heads", "dim", "vdim", "gate_cap"}}
Optional: "max_position_embeddings", "torch_dtype", "eos_token_id", "bos_token_id".

Checkpoint names: embed, head, final.norm{, .b, .alpha}; per layer l<i>.norm1{, .b, .alpha}, l<i>.norm2{...},
l<i>.mlp.{gate, up, down}, and under l<i>.mix: {in, conv, conv.b, x, dt, dt.b, A_log, D, o} |
{q, q.b, k, k.b, v, v.b, g, o} | left.{q, k, v, q.conv, k.conv, v.conv, o, out},
right.{q, k, v, g, i, i.b, f, f.b, norm, o, out}.
"""
import json
from dataclasses import dataclass
from typing import Any, Dict, Tuple

from ..config.model_config import ArchConfig, ConfigError
from ..config.registry import register_architecture
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

DEFAULT_MAX_POSITIONS = 131072


def _need(d: Any, key: str, where: str, kind=(int,), positive: bool = True):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError("config.json: %s lacks %r" % (where, key))
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, kind):
        raise ConfigError("config.json: %s.%s is %r" % (where, key, v))
    if positive and not v > 0:
        raise ConfigError("config.json: %s.%s must be > 0, is %r" % (where, key, v))
    return v


_NUMBER = (int, float)


def _check_heads(m: Any, where: str, kv: bool) -> None:
    heads = _need(m, "heads", where)
    _need(m, "dim", where)
    _need(m, "vdim", where)
    if kv:
        g = _need(m, "kv_heads", where)
        if heads % g:
            raise ConfigError("config.json: %s.heads %d is not a multiple of kv_heads %d" % (where, heads, g))
        _need(m, "scale", where, _NUMBER)


@dataclass(frozen=True)
class NiresunConfig(ArchConfig):
    width: int = 0
    norm_eps: float = 1e-5
    layers_json: str = "[]"        # the "layers" list as it was read (text: the dataclass is frozen and hashable)

    ARCHITECTURE = "Niresun"

    @property
    def layers(self) -> Tuple[Dict[str, Any], ...]:
        return tuple(json.loads(self.layers_json))

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "NiresunConfig":
        vocab = _need(d, "vocab", "the configuration")
        width = _need(d, "width", "the configuration")
        eps = _need(d.get("norm"), "eps", "norm", _NUMBER)
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        cfg = cls(architecture=cls.ARCHITECTURE, vocab_size=int(vocab),
                  max_position_embeddings=int(d.get("max_position_embeddings") or DEFAULT_MAX_POSITIONS),
                  torch_dtype=str(d.get("torch_dtype") or "bfloat16"), eos_token_ids=eos_ids,
                  bos_token_id=None if d.get("bos_token_id") is None else int(d["bos_token_id"]),
                  width=int(width), norm_eps=float(eps), layers_json=json.dumps(layers))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for i, layer in enumerate(self.layers):
            where = "layers[%d]" % i
            kind = layer.get("type") if isinstance(layer, dict) else None
            m = layer.get("mixer") if isinstance(layer, dict) else None
            at = where + ".mixer"
            if kind == "mamba1":
                for key in ("inner", "state", "dt_rank", "conv"):
                    _need(m, key, at)
            elif kind == "attention":
                _check_heads(m, at, kv=True)
                rot = m.get("rot")
                if rot is not None:
                    _need(rot, "base", at + ".rot", _NUMBER)
                    dims = _need(rot, "dims", at + ".rot")
                    if dims % 2 or dims > m["dim"]:
                        raise ConfigError("config.json: %s.rot.dims %d must be even and at most dim %d" % (at, dims, m["dim"]))
                    sc = rot.get("scaling")
                    if sc is not None:
                        for key in ("factor", "low", "high", "original"):
                            _need(sc, key, at + ".rot.scaling", _NUMBER)
                        if sc["high"] == sc["low"]:
                            raise ConfigError("config.json: %s.rot.scaling.high equals low" % at)
                if m.get("mask") is not None:
                    _need(m["mask"], "size", at + ".mask")
            elif kind == "parallel":
                left, right = (m or {}).get("left"), (m or {}).get("right")
                _check_heads(left, at + ".left", kv=True)
                _need(left, "conv", at + ".left")
                if left.get("q_temp") is not None:
                    _need(left["q_temp"], "coef", at + ".left.q_temp", _NUMBER, positive=False)
                    _need(left["q_temp"], "every", at + ".left.q_temp")
                _check_heads(right, at + ".right", kv=False)
                _need(right, "gate_cap", at + ".right", _NUMBER)
            else:
                raise ConfigError("config.json: %s.type %r is not supported (mamba1, attention, parallel)" % (where, kind))
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError("config.json: %s.mlp.kind %r is not supported (dense)"
                                      % (where, mlp.get("kind") if isinstance(mlp, dict) else mlp))
                _need(mlp, "ff", where + ".mlp")

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.ARCHITECTURE, "vocab": self.vocab_size, "width": self.width,
                "norm": {"eps": self.norm_eps}, "layers": list(self.layers),
                "max_position_embeddings": self.max_position_embeddings, "torch_dtype": self.torch_dtype,
                "eos_token_id": list(self.eos_token_ids) or None, "bos_token_id": self.bos_token_id}


def _mixer_spec(kind: str, m: Dict[str, Any], W: int, eps: float) -> PartSpec:
    if kind == "mamba1":
        return PartSpec("selective_scan", {"prefix": "mix", "hidden_size": W, "inner": m["inner"], "state": m["state"],
                                           "dt_rank": m["dt_rank"], "conv": m["conv"]})
    if kind == "attention":
        position = None
        rot = m.get("rot")
        if rot is not None:
            sc = rot.get("scaling")
            scaling = None if sc is None else {"rope_type": "llama3", "factor": sc["factor"], "low_freq_factor": sc["low"],
                                               "high_freq_factor": sc["high"],
                                               "original_max_position_embeddings": sc["original"]}
            position = PartSpec("rotary", {"head_dim": m["dim"], "rotary_dim": rot["dims"], "theta": rot["base"],
                                           "scaling": scaling, "style": "neox"})
        mask = m.get("mask")
        return PartSpec("flex_attention", {
            "prefix": "mix", "hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"],
            "head_dim": m["dim"], "v_head_dim": m["vdim"], "scale": m["scale"], "position": position, "qkv_bias": True,
            "chunk": mask["size"] if mask else None, "output_gate": True})
    left, right = m["left"], m["right"]
    temp = left.get("q_temp") or {}
    return PartSpec("parallel_pair", {
        "prefix": "mix", "hidden_size": W, "eps": eps, "scale": 0.5,
        "left": PartSpec("flex_attention", {
            "hidden_size": W, "num_heads": left["heads"], "num_kv_heads": left["kv_heads"], "head_dim": left["dim"],
            "v_head_dim": left["vdim"], "scale": left["scale"], "conv_taps": left["conv"], "unit_norm_eps": eps,
            "temp_coef": temp.get("coef", 0.0), "temp_every": temp.get("every", 0)}),
        "right": PartSpec("matrix_memory", {"hidden_size": W, "heads": right["heads"], "dim": right["dim"],
                                            "vdim": right["vdim"], "gate_cap": right["gate_cap"], "eps": eps})})


def build_niresun_spec(cfg: NiresunConfig) -> ModelSpec:
    W = cfg.width

    def norm(name: str) -> PartSpec:
        return PartSpec("dynamic_tanh", {"prefix": name, "size": W, "weight_name": "", "bias_name": "b",
                                         "alpha_name": "alpha"})

    layers, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        mlp = layer.get("mlp")
        norms = {"input": norm("norm1")}
        if mlp is None:
            ffn = PartSpec("none", {})
        else:
            norms["post_mixer"] = norm("norm2")
            ffn = PartSpec("gated_mlp", {"prefix": "mlp", "hidden_size": W, "intermediate_size": mlp["ff"],
                                         "activation": "gelu_tanh", "gate_name": "gate", "up_name": "up",
                                         "down_name": "down", "bare_names": True})
        layers.append(LayerSpec(prefix="l%d" % i, block=PartSpec("prenorm_residual"),
                                mixer=_mixer_spec(layer["type"], layer["mixer"], W, cfg.norm_eps), feed_forward=ffn,
                                norms=norms))
        schedule.append(ScheduleEntry(i))
    return ModelSpec(
        embedding=PartSpec("token_embedding", {"prefix": "embed", "vocab_size": cfg.vocab_size, "hidden_size": W,
                                               "weight_name": ""}),
        layers=tuple(layers), schedule=tuple(schedule), final_norm=norm("final.norm"),
        head=PartSpec("lm_head", {"prefix": "head", "vocab_size": cfg.vocab_size, "hidden_size": W,
                                  "weight_name": "head"}),
        vocab_size=cfg.vocab_size, hidden_size=W)


register_architecture("Niresun", "niresun", NiresunConfig, build_niresun_spec)
