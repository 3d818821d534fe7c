"""Zevetar as a ModelSpec: a decoder whose layers run their mixer and their feed-forward side by side.

Every layer: h = rms_norm(x), x += ls1 * mixer(h) + ls2 * ffn(h) (one norm, both sublayers read it, each result scaled
entry by entry by a vector of the layer). The mixer is one of
- "latent_attention": softmax attention over a cached latent (parts/latent_attention.py) with a gate for every entry
  of the heads' values, rotation of interleaved pairs with YaRN scaling of the frequencies, a sliding window; a layer
  may read an earlier layer's latent (``kv_from``);
- "retention": linear attention with a fixed decay per head and a state per request (parts/retention.py).
The feed-forward is dense and gated (SiLU), or experts chosen by a sigmoid router whose scores weigh the experts'
inputs, with a shared expert behind a gate of one number a token (parts/routed_moe.py), or absent. The embedding is
scaled; the logits come from the embedding table itself, are scaled and then bounded by a soft cap. The reference has
no such architecture; its model files hard-wire Llama's block (core/src/model_executor/models/llama/llama.rs:276-385).

config.json: "architecture": "Zevetar", "vocab", "width", "norm": {"eps"}, "embedding": {"scale"}, "logit_scale",
"logit_softcap", and "layers", a list of {"type", "mixer", "mlp"} with
  latent_attention: {"heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank", "scale", "rot": {"base", "dims",
                     "scaling"?: {"factor", "original", "fast", "slow"}}, "mask"?: {"size"}, "kv_from"?}
  retention:        {"heads", "dim", "vdim", "decay": [one per head], "rot"?: {"base", "dims"}}
  mlp: null | {"kind": "dense", "ff"} | {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"},
               "shared"?: {"ff"}}
Optional: "max_position_embeddings", "torch_dtype", "eos_token_id", "bos_token_id".

Checkpoint names: embed, final.norm; per layer l<i>.{norm1, ls1, ls2}, l<i>.mix.{dq, dq.norm, uq, dkv, dkv.norm, uk,
uv, g, o} or l<i>.mix.{q, k, v, g, o}, l<i>.mlp.{gate, up, down} or l<i>.mlp.{router, e<k>.{gate, up, down},
shared.{gate, up, down, sg}}.
"""
import json
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..config.model_config import ArchConfig, ConfigError
from ..config.registry import register_architecture
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

DEFAULT_MAX_POSITIONS = 131072
_NUMBER = (int, float)


def _need(d: Any, key: str, where: str, kind=(int,), positive: bool = True):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError("config.json: %s lacks %r" % (where, key))
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, kind):
        raise ConfigError("config.json: %s.%s is %r" % (where, key, v))
    if positive and not v > 0:
        raise ConfigError("config.json: %s.%s must be > 0, is %r" % (where, key, v))
    return v


def _check_rot(rot: Any, where: str, limit: int, scaling_ok: bool):
    _need(rot, "base", where, _NUMBER)
    dims = _need(rot, "dims", where)
    if dims % 2 or dims > limit:
        raise ConfigError("config.json: %s.dims %d must be even and at most %d" % (where, dims, limit))
    sc = rot.get("scaling")
    if sc is not None:
        if not scaling_ok:
            raise ConfigError("config.json: %s.scaling is not supported here" % where)
        for key in ("factor", "original", "fast", "slow"):
            _need(sc, key, where + ".scaling", _NUMBER)
    return (float(rot["base"]), dims, None if sc is None else tuple(sorted((k, float(v)) for k, v in sc.items())))


@dataclass(frozen=True)
class ZevetarConfig(ArchConfig):
    width: int = 0
    norm_eps: float = 1e-5
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: float = 0.0
    layers_json: str = "[]"        # the "layers" list as it was read (text: the dataclass is frozen and hashable)

    ARCHITECTURE = "Zevetar"

    @property
    def layers(self) -> Tuple[Dict[str, Any], ...]:
        return tuple(json.loads(self.layers_json))

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "ZevetarConfig":
        vocab = _need(d, "vocab", "the configuration")
        width = _need(d, "width", "the configuration")
        eps = _need(d.get("norm"), "eps", "norm", _NUMBER)
        emb = d.get("embedding")
        emb_scale = 1.0 if emb is None else _need(emb, "scale", "embedding", _NUMBER, positive=False)
        logit_scale = _need(d, "logit_scale", "the configuration", _NUMBER, positive=False) if "logit_scale" in d else 1.0
        cap = d.get("logit_softcap")
        if cap is not None:
            cap = _need(d, "logit_softcap", "the configuration", _NUMBER)
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        cfg = cls(architecture=cls.ARCHITECTURE, vocab_size=int(vocab),
                  max_position_embeddings=int(d.get("max_position_embeddings") or DEFAULT_MAX_POSITIONS),
                  torch_dtype=str(d.get("torch_dtype") or "bfloat16"), eos_token_ids=eos_ids,
                  bos_token_id=None if d.get("bos_token_id") is None else int(d["bos_token_id"]),
                  width=int(width), norm_eps=float(eps), embedding_scale=float(emb_scale),
                  logit_scale=float(logit_scale), logit_softcap=float(cap or 0.0), layers_json=json.dumps(layers))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        owners = {}
        for i, layer in enumerate(self.layers):
            where = "layers[%d]" % i
            kind = layer.get("type") if isinstance(layer, dict) else None
            m = layer.get("mixer") if isinstance(layer, dict) else None
            at = where + ".mixer"
            if kind == "latent_attention":
                for key in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"):
                    _need(m, key, at)
                _need(m, "scale", at, _NUMBER)
                rot = _check_rot(m.get("rot"), at + ".rot", m["rot_dim"], scaling_ok=True)
                if m.get("mask") is not None:
                    _need(m["mask"], "size", at + ".mask")
                src = m.get("kv_from")
                mine = (m["kv_rank"], m["rot_dim"]) + rot
                if src is None:
                    owners[i] = mine
                else:
                    if isinstance(src, bool) or not isinstance(src, int) or src not in owners:
                        raise ConfigError("config.json: %s.kv_from %r names no earlier layer with a latent of its own"
                                          % (at, src))
                    if owners[src] != mine:
                        raise ConfigError("config.json: %s reads the latent of layer %d, whose sizes or rotation differ"
                                          % (at, src))
            elif kind == "retention":
                heads = _need(m, "heads", at)
                _need(m, "dim", at)
                _need(m, "vdim", at)
                decay = m.get("decay")
                if not isinstance(decay, list) or len(decay) != heads or any(
                        isinstance(g, bool) or not isinstance(g, _NUMBER) or not (0 <= g <= 1) for g in decay):
                    raise ConfigError("config.json: %s.decay must list %d numbers within [0, 1]" % (at, heads))
                if m.get("rot") is not None:
                    _check_rot(m["rot"], at + ".rot", m["dim"], scaling_ok=False)
            else:
                raise ConfigError("config.json: %s.type %r is not supported (latent_attention, retention)" % (where, kind))
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            mk = mlp.get("kind") if isinstance(mlp, dict) else None
            if mk == "dense":
                _need(mlp, "ff", where + ".mlp")
            elif mk == "moe":
                _need(mlp.get("expert"), "ff", where + ".mlp.expert")
                e = _need(mlp.get("router"), "experts", where + ".mlp.router")
                top = _need(mlp.get("router"), "top", where + ".mlp.router")
                if top > e:
                    raise ConfigError("config.json: %s.mlp.router.top %d exceeds experts %d" % (where, top, e))
                if mlp.get("shared") is not None:
                    _need(mlp["shared"], "ff", where + ".mlp.shared")
            else:
                raise ConfigError("config.json: %s.mlp.kind %r is not supported (dense, moe)" % (where, mk))

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.ARCHITECTURE, "vocab": self.vocab_size, "width": self.width,
                "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
                "logit_scale": self.logit_scale, "logit_softcap": self.logit_softcap or None,
                "layers": list(self.layers), "max_position_embeddings": self.max_position_embeddings,
                "torch_dtype": self.torch_dtype, "eos_token_id": list(self.eos_token_ids) or None,
                "bos_token_id": self.bos_token_id}


def _rotary(rot: Dict[str, Any], head_dim: int, style: str) -> PartSpec:
    sc = rot.get("scaling")
    scaling = None if sc is None else {"rope_type": "yarn", "factor": sc["factor"], "beta_fast": sc["fast"],
                                       "beta_slow": sc["slow"], "original_max_position_embeddings": sc["original"]}
    return PartSpec("rotary", {"head_dim": head_dim, "rotary_dim": rot["dims"], "theta": rot["base"],
                               "scaling": scaling, "style": style})


def build_zevetar_spec(cfg: ZevetarConfig) -> ModelSpec:
    W = cfg.width
    layers_cfg = cfg.layers

    def norm(name: str) -> PartSpec:
        return PartSpec("rms_norm", {"prefix": name, "size": W, "eps": cfg.norm_eps, "weight_name": ""})

    def gated(prefix: str, ff: int) -> PartSpec:
        return PartSpec("gated_mlp", {"prefix": prefix, "hidden_size": W, "intermediate_size": ff, "activation": "silu",
                                      "gate_name": "gate", "up_name": "up", "down_name": "down", "bare_names": True})

    # the pages of a latent are kept for the widest window among the layers that read them (all of them, if one of
    # these layers sees everything)
    kept: Dict[int, Optional[int]] = {}
    for i, layer in enumerate(layers_cfg):
        if layer["type"] != "latent_attention":
            continue
        m = layer["mixer"]
        owner = m.get("kv_from", i) if m.get("kv_from") is not None else i
        size = (m.get("mask") or {}).get("size")
        if owner not in kept:
            kept[owner] = size
        elif kept[owner] is not None:
            kept[owner] = None if size is None else max(kept[owner], size)

    layers, schedule = [], []
    for i, layer in enumerate(layers_cfg):
        m, mlp = layer["mixer"], layer.get("mlp")
        src: Optional[int] = None
        if layer["type"] == "latent_attention":
            src = m.get("kv_from")
            owner = i if src is None else src
            mixer = PartSpec("latent_attention", {
                "prefix": "mix", "hidden_size": W, "num_heads": m["heads"], "head_dim": m["dim"], "rot_dim": m["rot_dim"],
                "v_head_dim": m["vdim"], "kv_rank": m["kv_rank"], "q_rank": m["q_rank"], "scale": m["scale"],
                "eps": cfg.norm_eps, "owns_latent": src is None, "gate_per_entry": True, "weights_f32": True,
                "window": (m.get("mask") or {}).get("size"), "cache_window": kept[owner],
                "position": _rotary(m["rot"], m["rot_dim"], "gptj")})
        else:
            rot = m.get("rot")
            mixer = PartSpec("retention", {
                "prefix": "mix", "hidden_size": W, "heads": m["heads"], "dim": m["dim"], "vdim": m["vdim"],
                "decay": tuple(m["decay"]), "eps": cfg.norm_eps,
                "position": _rotary(rot, m["dim"], "neox") if rot is not None else None})
        if mlp is None:
            ffn = PartSpec("none", {})
        elif mlp["kind"] == "dense":
            ffn = gated("mlp", mlp["ff"])
        else:
            shared = mlp.get("shared")
            ffn = PartSpec("routed_moe", {
                "prefix": "mlp", "hidden_size": W, "expert_size": mlp["expert"]["ff"],
                "num_experts": mlp["router"]["experts"], "top": mlp["router"]["top"],
                "shared": gated("shared", shared["ff"]) if shared is not None else None,
                "shared_gate": "shared.sg" if shared is not None else None})
        layers.append(LayerSpec(prefix="l%d" % i, block=PartSpec("parallel_scaled", {"hidden_size": W}), mixer=mixer,
                                feed_forward=ffn, norms={"input": norm("norm1")}))
        schedule.append(ScheduleEntry(i, cache_from=src))
    return ModelSpec(
        embedding=PartSpec("token_embedding", {"prefix": "embed", "vocab_size": cfg.vocab_size, "hidden_size": W,
                                               "weight_name": "", "scale": cfg.embedding_scale}),
        layers=tuple(layers), schedule=tuple(schedule), final_norm=norm("final.norm"),
        head=PartSpec("lm_head", {"prefix": "head", "vocab_size": cfg.vocab_size, "hidden_size": W,
                                  "weight_name": "embed", "logit_scale": cfg.logit_scale,
                                  "softcap": cfg.logit_softcap}),
        vocab_size=cfg.vocab_size, hidden_size=W)


# a layer without a feed-forward may still carry the scale of one
ZEVETAR_TOLERATED = (".ls2",)

register_architecture("Zevetar", "zevetar", ZevetarConfig, build_zevetar_spec, tolerated_tensors=ZEVETAR_TOLERATED)
