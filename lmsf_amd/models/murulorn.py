"""Murulorn as a ModelSpec: a decoder with a loop over some of its layers, norms around every sublayer and inputs from
the token itself at every layer.

The embedding adds a row of a hashed pair table (previous token, token) to the token's own row. Every layer:
x += n1b(mixer(n1(x))); x += n2b(ffn(n2(x))); x += side(x, token), every n an RMS norm whose stored weight w acts as
1 + w, side a small gated product with a slice of a per-token table. Layers ``loop.start`` to ``loop.stop`` - 1 run
``loop.times`` times in a row with the same weights and a cache or state per pass; every pass begins with
x = W_in [x ; x0], x0 the embedding's output. The mixer is one of
- "attention": softmax attention within a window, one norm over all of q and one over all of k, partial rotation of
  interleaved pairs, values normed per head and rotated over their whole width, scores bounded by a soft cap, one
  sigmoid gate a head (parts/normed_attention.py);
- "channel_delta": the gated delta rule with a decay per head and key channel (parts/delta_rule.py).
The feed-forward is W_down relu(W_up h)^2, or experts of that form chosen by a softmax router within the best groups of
neighbouring experts, weighted by their scores as they are (parts/routed_moe.py), or absent. The logits come from the
embedding table behind the model's norm. The reference has no such architecture; its model files hard-wire Llama's
block (core/src/model_executor/models/llama/llama.rs:276-385).

config.json: "architecture": "Murulorn", "vocab", "width", "norm": {"eps"}, "embedding": {"bigram": {"buckets",
"mul_prev", "mul_cur"}}, "token_side"?: {"dim"}, "loop"?: {"start", "stop", "times"}, and "layers", a list of
{"type", "mixer", "mlp"} with
  attention:     {"heads", "kv_heads", "dim", "vdim", "scale", "softcap"?, "rot": {"base", "dims"}, "mask": {"size"}}
  channel_delta: {"heads", "kv_heads", "dim", "vdim", "conv", "decay_rank"?, "gate_rank"?}
  mlp: null | {"kind": "dense", "ff"} | {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top", "groups"?:
               {"count", "keep"}}}
The two ranks are the rows of the tensors l<i>.mix.a1 and l<i>.mix.g1; a checkpoint's header gives them where
config.json does not (``complete_from_checkpoint``), and without a checkpoint they default to the width of a key.
Optional: "max_position_embeddings", "torch_dtype", "eos_token_id", "bos_token_id".

Checkpoint names: embed, bigram, loop.in, side.embed, final.norm; per layer l<i>.{norm1, norm1b, norm2, norm2b},
l<i>.side.{gate, proj, norm}, l<i>.mix.{q, k, v, q.norm, k.norm, g, o} or l<i>.mix.{q, k, v, q.conv, k.conv, v.conv, b,
A_log, a1, a2, dt_bias, g1, g2, norm, o}, l<i>.mlp.{up, down} or l<i>.mlp.{router, e<k>.{up, down}}.
"""
import json
import os
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

from ..config.model_config import ArchConfig, ConfigError
from ..config.registry import register_architecture
from ..parts.base import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

DEFAULT_MAX_POSITIONS = 131072
_NUMBER = (int, float)


def _need(d: Any, key: str, where: str, kind=(int,), positive: bool = True, at_least: Optional[int] = None):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError("config.json: %s lacks %r" % (where, key))
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, kind):
        raise ConfigError("config.json: %s.%s is %r" % (where, key, v))
    if at_least is not None:
        if v < at_least:
            raise ConfigError("config.json: %s.%s must be >= %d, is %r" % (where, key, at_least, v))
    elif positive and not v > 0:
        raise ConfigError("config.json: %s.%s must be > 0, is %r" % (where, key, v))
    return v


def _header_shapes(folder: str) -> Dict[str, Tuple[int, ...]]:
    """Names and shapes of a folder's checkpoint tensors, from the files' headers alone."""
    from ..weights.loader import list_weight_files
    from ..weights.safetensors_io import SafetensorsFile
    shapes: Dict[str, Tuple[int, ...]] = {}
    for path in list_weight_files(folder):
        f = SafetensorsFile(path)
        try:
            for name, e in f.entries.items():
                shapes[name] = tuple(e.shape)
        finally:
            f.close()
    return shapes


@dataclass(frozen=True)
class MurulornConfig(ArchConfig):
    width: int = 0
    norm_eps: float = 1e-5
    buckets: int = 1
    mul_prev: int = 0
    mul_cur: int = 0
    side_dim: int = 0               # 0: no input from the token at the layers
    loop_start: int = 0
    loop_stop: int = 0              # start == stop: no loop
    loop_times: int = 1
    layers_json: str = "[]"         # the "layers" list as it was read (text: the dataclass is frozen and hashable)

    ARCHITECTURE = "Murulorn"

    @property
    def layers(self) -> Tuple[Dict[str, Any], ...]:
        return tuple(json.loads(self.layers_json))

    @staticmethod
    def complete_from_checkpoint(d: Dict[str, Any], folder: str) -> Dict[str, Any]:
        """The ranks of the decay's and the gate's low-rank products, where config.json does not name them, are the
        rows of the tensors that hold them."""
        layers = d.get("layers")
        if not isinstance(layers, list):
            return d
        lacking = [i for i, layer in enumerate(layers) if isinstance(layer, dict) and layer.get("type") == "channel_delta"
                   and isinstance(layer.get("mixer"), dict)
                   and not ("decay_rank" in layer["mixer"] and "gate_rank" in layer["mixer"])]
        if not lacking:
            return d
        try:
            shapes = _header_shapes(folder)
        except Exception:  # noqa: BLE001 - no checkpoint (random weights): the defaults stand
            return d
        d = json.loads(json.dumps(d))
        for i in lacking:
            m = d["layers"][i]["mixer"]
            for key, name in (("decay_rank", "l%d.mix.a1" % i), ("gate_rank", "l%d.mix.g1" % i)):
                if key not in m and name in shapes and len(shapes[name]) == 2:
                    m[key] = int(shapes[name][0])
        return d

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MurulornConfig":
        vocab = _need(d, "vocab", "the configuration")
        width = _need(d, "width", "the configuration")
        eps = _need(d.get("norm"), "eps", "norm", _NUMBER)
        big = (d.get("embedding") or {}).get("bigram") if isinstance(d.get("embedding"), dict) else None
        buckets = _need(big, "buckets", "embedding.bigram")
        mul_prev = _need(big, "mul_prev", "embedding.bigram", at_least=0)
        mul_cur = _need(big, "mul_cur", "embedding.bigram", at_least=0)
        side = d.get("token_side")
        side_dim = 0 if side is None else _need(side, "dim", "token_side")
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        loop = d.get("loop")
        start = stop = 0
        times = 1
        if loop is not None:
            start = _need(loop, "start", "loop", at_least=0)
            stop = _need(loop, "stop", "loop", at_least=0)
            times = _need(loop, "times", "loop")
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        cfg = cls(architecture=cls.ARCHITECTURE, vocab_size=int(vocab),
                  max_position_embeddings=int(d.get("max_position_embeddings") or DEFAULT_MAX_POSITIONS),
                  torch_dtype=str(d.get("torch_dtype") or "bfloat16"), eos_token_ids=eos_ids,
                  bos_token_id=None if d.get("bos_token_id") is None else int(d["bos_token_id"]),
                  width=int(width), norm_eps=float(eps), buckets=int(buckets), mul_prev=int(mul_prev),
                  mul_cur=int(mul_cur), side_dim=int(side_dim), loop_start=int(start), loop_stop=int(stop),
                  loop_times=int(times), layers_json=json.dumps(layers))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        layers = self.layers
        if not (0 <= self.loop_start <= self.loop_stop <= len(layers)):
            raise ConfigError("config.json: loop %d to %d does not lie within the %d layers"
                              % (self.loop_start, self.loop_stop, len(layers)))
        for i, layer in enumerate(layers):
            where = "layers[%d]" % i
            kind = layer.get("type") if isinstance(layer, dict) else None
            m = layer.get("mixer") if isinstance(layer, dict) else None
            at = where + ".mixer"
            if kind not in ("attention", "channel_delta"):
                raise ConfigError("config.json: %s.type %r is not supported (attention, channel_delta)" % (where, kind))
            heads, kv = _need(m, "heads", at), _need(m, "kv_heads", at)
            if heads % kv:
                raise ConfigError("config.json: %s.heads %d is not a multiple of kv_heads %d" % (at, heads, kv))
            dim, vdim = _need(m, "dim", at), _need(m, "vdim", at)
            if kind == "attention":
                if dim % 2 or vdim % 2:
                    raise ConfigError("config.json: %s.dim and .vdim must be even, are %d and %d" % (at, dim, vdim))
                _need(m, "scale", at, _NUMBER)
                if m.get("softcap") is not None:
                    _need(m, "softcap", at, _NUMBER)
                _need(m.get("rot"), "base", at + ".rot", _NUMBER)
                dims = _need(m.get("rot"), "dims", at + ".rot")
                if dims % 2 or dims > dim:
                    raise ConfigError("config.json: %s.rot.dims %d must be even and at most %d" % (at, dims, dim))
                _need(m.get("mask"), "size", at + ".mask")
            else:
                _need(m, "conv", at)
                if dim > 256:
                    raise ConfigError("config.json: %s.dim %d: keys of at most 256 entries" % (at, dim))
                for key in ("decay_rank", "gate_rank"):
                    if key in m:
                        _need(m, key, at)
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            mk = mlp.get("kind") if isinstance(mlp, dict) else None
            if mk == "dense":
                _need(mlp, "ff", where + ".mlp")
            elif mk == "moe":
                _need(mlp.get("expert"), "ff", where + ".mlp.expert")
                r = mlp.get("router")
                e = _need(r, "experts", where + ".mlp.router")
                top = _need(r, "top", where + ".mlp.router")
                count = keep = 1
                if r.get("groups") is not None:
                    count = _need(r["groups"], "count", where + ".mlp.router.groups")
                    keep = _need(r["groups"], "keep", where + ".mlp.router.groups")
                if e % count or keep > count or keep * (e // count) < top or top > e:
                    raise ConfigError("config.json: %s.mlp.router: %d of %d experts from %d of %d groups"
                                      % (where, top, e, keep, count))
            else:
                raise ConfigError("config.json: %s.mlp.kind %r is not supported (dense, moe)" % (where, mk))

    def to_dict(self) -> Dict[str, Any]:
        out = {"architecture": self.ARCHITECTURE, "vocab": self.vocab_size, "width": self.width,
               "norm": {"eps": self.norm_eps},
               "embedding": {"bigram": {"buckets": self.buckets, "mul_prev": self.mul_prev, "mul_cur": self.mul_cur}},
               "layers": list(self.layers), "max_position_embeddings": self.max_position_embeddings,
               "torch_dtype": self.torch_dtype, "eos_token_id": list(self.eos_token_ids) or None,
               "bos_token_id": self.bos_token_id}
        if self.side_dim:
            out["token_side"] = {"dim": self.side_dim}
        if self.loop_stop > self.loop_start:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        return out


def layer_runs(cfg: MurulornConfig) -> List[int]:
    """The layers in the order in which they run."""
    n = len(cfg.layers)
    a, b = cfg.loop_start, cfg.loop_stop
    return list(range(a)) + list(range(a, b)) * cfg.loop_times + list(range(b, n))


def build_murulorn_spec(cfg: MurulornConfig) -> ModelSpec:
    W = cfg.width
    layers_cfg = cfg.layers
    looped = cfg.loop_stop > cfg.loop_start

    def norm(name: str) -> PartSpec:
        return PartSpec("group_rms_norm", {"prefix": name, "size": W, "eps": cfg.norm_eps, "weight_name": "",
                                           "weight_offset": 1.0})

    def rotary(width: int, dims: int, base: float) -> PartSpec:
        return PartSpec("rotary", {"head_dim": width, "rotary_dim": dims, "theta": base, "style": "gptj",
                                   "angles": "float64"})

    layers = []
    for i, layer in enumerate(layers_cfg):
        m, mlp = layer["mixer"], layer.get("mlp")
        if layer["type"] == "attention":
            mixer = PartSpec("normed_attention", {
                "prefix": "mix", "hidden_size": W, "num_heads": m["heads"], "num_kv_heads": m["kv_heads"],
                "head_dim": m["dim"], "v_head_dim": m["vdim"], "scale": m["scale"], "eps": cfg.norm_eps,
                "softcap": m.get("softcap") or 0.0, "window": m["mask"]["size"],
                "position": rotary(m["dim"], m["rot"]["dims"], m["rot"]["base"]),
                "value_position": rotary(m["vdim"], m["vdim"], m["rot"]["base"])})
        else:
            mixer = PartSpec("gated_delta", {
                "prefix": "mix", "hidden_size": W, "heads": m["heads"], "kv_heads": m["kv_heads"], "dim": m["dim"],
                "vdim": m["vdim"], "conv": m["conv"], "decay_rank": m.get("decay_rank", m["dim"]),
                "gate_rank": m.get("gate_rank", m["dim"]), "eps": cfg.norm_eps})
        if mlp is None:
            ffn = PartSpec("none", {})
        elif mlp["kind"] == "dense":
            ffn = PartSpec("plain_mlp", {"prefix": "mlp", "hidden_size": W, "intermediate_size": mlp["ff"],
                                         "activation": "relu_squared"})
        else:
            r = mlp["router"]
            g = r.get("groups") or {"count": 1, "keep": 1}
            ffn = PartSpec("routed_moe", {
                "prefix": "mlp", "hidden_size": W, "expert_size": mlp["expert"]["ff"], "num_experts": r["experts"],
                "top": r["top"], "gated": False, "scores": "softmax", "groups": g["count"], "keep_groups": g["keep"],
                "weight_on": "output"})
        block = {"hidden_size": W}
        if looped and i == cfg.loop_start:
            block["inject"] = "loop.in"
        if cfg.side_dim:
            block["side"] = {"prefix": "side", "dim": cfg.side_dim, "at": i * cfg.side_dim, "table_name": "side.embed",
                             "table_width": len(layers_cfg) * cfg.side_dim, "vocab_size": cfg.vocab_size,
                             "eps": cfg.norm_eps}
        norms = {"pre_mixer": norm("norm1"), "post_mixer": norm("norm1b")}
        if mlp is not None:
            norms.update({"pre_ffn": norm("norm2"), "post_ffn": norm("norm2b")})
        layers.append(LayerSpec(prefix="l%d" % i, block=PartSpec("sandwich", block), mixer=mixer, feed_forward=ffn,
                                norms=norms))
    return ModelSpec(
        embedding=PartSpec("hashed_pair_embedding", {
            "prefix": "embed", "vocab_size": cfg.vocab_size, "hidden_size": W, "buckets": cfg.buckets,
            "mul_prev": cfg.mul_prev, "mul_cur": cfg.mul_cur, "pair_name": "bigram", "keep_output": looped}),
        layers=tuple(layers), schedule=tuple(ScheduleEntry(i) for i in layer_runs(cfg)),
        final_norm=norm("final.norm"),
        head=PartSpec("lm_head", {"prefix": "head", "vocab_size": cfg.vocab_size, "hidden_size": W,
                                  "weight_name": "embed"}),
        vocab_size=cfg.vocab_size, hidden_size=W)


# a layer without a feed-forward may still carry the norms of one; a model without a loop its matrix
MURULORN_TOLERATED = (".norm2", ".norm2b", "loop.in")

register_architecture("Murulorn", "murulorn", MurulornConfig, build_murulorn_spec,
                      tolerated_tensors=MURULORN_TOLERATED)
