"""Nodutar: a decoder whose layers put a norm before and behind each branch,
x <- x + N1b(mixer(N1(x))), x <- x + N2b(ff(N2(x))), with RMS norms whose gain is one plus the stored weight; a run of
consecutive layers may be passed several times with the same weights, every pass with a cache and state of its
own and the embedding output added to the stream in front of every pass but the first.  A mixer is softmax
attention whose values are its keys as projected, with unit-normed queries and keys and a logarithmic penalty
on distance ("attention"), or chunked attention with normed and partly rotated queries and keys and rotated
values beside a gated linear recurrence, scaled and summed ("parallel").  A feed-forward is a mixture of
silu-gated experts with a biased router.  The head is the embedding table.

config.json: `architecture` = "Nodutar"; `vocab`, `width`; `norm` = {eps}; `loop` = {start, stop, times} or
absent; `layers`, a list of {type: "attention" | "parallel", mixer: {...}, mlp: {...} or null}.
Mixer sizes: attention {heads, kv_heads, dim, vdim, scale}; parallel {left: {heads, kv_heads, dim, vdim, scale,
mask: {size}, rot: {base, dims}}, right: {heads, dim, vdim}, left_scale, right_scale}.
mlp: {kind: "moe", expert: {ff}, router: {experts, top}}.
Tensors: embed, l<i>.norm1, norm1b, norm2, norm2b, l<i>.mix.*, l<i>.mlp.*, final.norm.
"""
from __future__ import annotations

import copy
import math
from typing import Any, Dict, List, Optional, Tuple

from .base import ConfigError, KeyReader
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, RunEntry

ARCHITECTURE = "Nodutar"
MIXER_TYPES = ("attention", "parallel")
MAX_POSITIONS = 1 << 20      # the design names no bound; rotation tables grow on demand up to here


def _attention_sizes(raw: Any, where: str, chunked: bool) -> Dict[str, Any]:
    r = KeyReader(raw, where)
    out = dict(heads=r.integer("heads"), kv_heads=r.integer("kv_heads"), dim=r.integer("dim"), vdim=r.integer("vdim"),
               scale=r.number("scale"))
    if out["heads"] % out["kv_heads"]:
        raise ConfigError(f"{where}: 'heads' {out['heads']} is not a multiple of 'kv_heads' {out['kv_heads']}")
    if not chunked:
        if out["vdim"] != out["dim"]:
            raise ConfigError(f"{where}: the keys serve as values, so 'vdim' {out['vdim']} must equal 'dim' {out['dim']}")
        return out
    out["mask"] = dict(size=KeyReader(r.raw_value("mask") or {}, where + ".mask").integer("size"))
    k = KeyReader(r.raw_value("rot") or {}, where + ".rot")
    dims = k.integer("dims")
    if dims % 2 or dims > out["dim"]:
        raise ConfigError(f"{where}.rot: 'dims' must be even and at most dim {out['dim']}, found {dims}")
    if out["vdim"] % 2:
        raise ConfigError(f"{where}: 'vdim' {out['vdim']} must be even: the values are rotated in pairs")
    out["rot"] = dict(base=k.number("base"), dims=dims)
    return out


def _mixer_sizes(kind: str, raw: Any, where: str) -> Dict[str, Any]:
    if kind == "attention":
        return _attention_sizes(raw, where, chunked=False)
    r = KeyReader(raw, where)
    g = KeyReader(r.raw_value("right") or {}, where + ".right")
    return dict(left=_attention_sizes(r.raw_value("left"), where + ".left", chunked=True),
                right=dict(heads=g.integer("heads"), dim=g.integer("dim"), vdim=g.integer("vdim")),
                left_scale=r.number("left_scale", positive=False), right_scale=r.number("right_scale", positive=False))


def _mlp_sizes(raw: Any, where: str) -> Optional[Dict[str, Any]]:
    if raw is None:
        return None
    m = KeyReader(raw, where)
    kind = m.string("kind", default="moe")
    if kind != "moe":
        raise ConfigError(f"{where}: kind {kind!r} is not one of ['moe']")
    e = KeyReader(m.raw_value("expert") or {}, where + ".expert")
    r = KeyReader(m.raw_value("router") or {}, where + ".router")
    out = dict(kind="moe", expert=dict(ff=e.integer("ff")), router=dict(experts=r.integer("experts"), top=r.integer("top")))
    if out["router"]["top"] > out["router"]["experts"]:
        raise ConfigError(f"{where}.router: {out['router']['top']} of {out['router']['experts']} experts cannot be chosen")
    return out


class NodutarConfig:
    architecture = ARCHITECTURE

    def __init__(self, vocab: int, width: int, eps: float, layers: List[Dict[str, Any]],
                 loop: Optional[Dict[str, int]] = None, init_std: Optional[float] = None):
        self.vocab, self.width, self.eps = vocab, width, eps
        self.layers, self.loop = layers, loop
        self.init_std = init_std
        self._fan_in: Optional[Dict[str, int]] = None

    # ---------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "NodutarConfig":
        r = KeyReader(raw)
        vocab, width = r.integer("vocab"), r.integer("width")
        eps = KeyReader(r.raw_value("norm") or {}, "config.json: norm").number("eps")
        raw_layers = r.raw_value("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError(f"config.json: 'layers' must be a non-empty list, found {raw_layers!r}")
        layers: List[Dict[str, Any]] = []
        for i, entry in enumerate(raw_layers):
            where = f"config.json: layers[{i}]"
            e = KeyReader(entry, where)
            kind = e.string("type")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"{where}: type {kind!r} is not one of {list(MIXER_TYPES)}")
            layers.append(dict(type=kind, mixer=_mixer_sizes(kind, e.raw_value("mixer"), where + ".mixer"),
                               mlp=_mlp_sizes(e.raw_value("mlp"), where + ".mlp")))
        loop = r.raw_value("loop")
        if loop is not None:
            k = KeyReader(loop, "config.json: loop")
            loop = dict(start=k.integer("start", minimum=0), stop=k.integer("stop", minimum=0), times=k.integer("times"))
            if not loop["start"] <= loop["stop"] <= len(layers):
                raise ConfigError(f"config.json: loop {loop} does not lie inside the {len(layers)} layers")
        return cls(vocab, width, eps, layers, loop=loop, init_std=raw.get("init_std"))

    def to_dict(self) -> Dict[str, Any]:
        """A config.json that reads back to this configuration."""
        d = dict(architecture=ARCHITECTURE, vocab=self.vocab, width=self.width, norm=dict(eps=self.eps),
                 layers=copy.deepcopy(self.layers))
        if self.loop is not None:
            d["loop"] = dict(self.loop)
        if self.init_std is not None:
            d["init_std"] = self.init_std
        return d

    # ---------------------------------------------------------------- description
    def _norm(self, name: str) -> PartSpec:
        return PartSpec("offset_rmsnorm", dict(size=self.width, eps=self.eps, weight=name))

    def _attention(self, m: Dict[str, Any], prefix: str, chunked: bool) -> PartSpec:
        names = {k: prefix + k for k in ("q", "k", "v", "o")}
        names.update(q_norm=prefix + "q.norm", k_norm=prefix + "k.norm")
        common = dict(hidden_size=self.width, n_heads=m["heads"], n_kv_heads=m["kv_heads"], dim=m["dim"], v_dim=m["vdim"],
                      scale=m["scale"], eps=self.eps, **names)
        if not chunked:
            return PartSpec("normed_attention", dict(common, values_from_keys=True, distance=(prefix + "r1", prefix + "r2")))
        rot = m["rot"]
        return PartSpec("normed_attention", dict(
            common, qk_gains=True, chunk=m["mask"]["size"],
            position=PartSpec("rope_pairs", dict(dims=rot["dims"], base=rot["base"], scaling=None,
                                                 max_positions=MAX_POSITIONS)),
            value_rotation=PartSpec("rope_pairs", dict(dims=m["vdim"], base=rot["base"], scaling=None,
                                                       max_positions=MAX_POSITIONS))))

    def _mixer(self, layer: Dict[str, Any]) -> PartSpec:
        m = layer["mixer"]
        if layer["type"] == "attention":
            return self._attention(m, "mix.", chunked=False)
        g = m["right"]
        right = PartSpec("gated_recurrence", dict(
            hidden_size=self.width, n_heads=g["heads"], dim=g["dim"], v_dim=g["vdim"], eps=self.eps, q="q", f="f",
            f_bias="f.b", lower="lower", v="v", norm="norm", o="o"))
        return PartSpec("side_by_side", dict(left=self._attention(m["left"], "", chunked=True), right=right,
                                             left_scale=m["left_scale"], right_scale=m["right_scale"],
                                             left_prefix="mix.left.", right_prefix="mix.right."))

    def _feed_forward(self, mlp: Dict[str, Any]) -> PartSpec:
        r = mlp["router"]
        return PartSpec("grouped_moe", dict(
            hidden_size=self.width, intermediate_size=mlp["expert"]["ff"], n_experts=r["experts"], top=r["top"],
            act="silu", router="mlp.router", router_bias="mlp.router.b", expert="mlp.e{}"))

    def run_order(self) -> List[Tuple[int, bool]]:
        """(layer, whether the embedding output joins the stream in front of it) as the layers run."""
        n = len(self.layers)
        if self.loop is None or self.loop["times"] <= 1 or self.loop["start"] == self.loop["stop"]:
            return [(i, False) for i in range(n)]
        start, stop = self.loop["start"], self.loop["stop"]
        order = [(i, False) for i in range(start)]
        for p in range(self.loop["times"]):
            order += [(i, p > 0 and i == start) for i in range(start, stop)]
        return order + [(i, False) for i in range(stop, n)]

    def model_spec(self) -> ModelSpec:
        blocks = []
        for i, layer in enumerate(self.layers):
            norms = {"mixer": self._norm("norm1"), "mixer_out": self._norm("norm1b")}
            ffn = None
            if layer["mlp"] is not None:
                ffn = self._feed_forward(layer["mlp"])
                norms.update(feed_forward=self._norm("norm2"), feed_forward_out=self._norm("norm2b"))
            blocks.append(BlockSpec(kind="sandwich", prefix=f"l{i}.", mixer=self._mixer(layer), feed_forward=ffn,
                                    norms=norms))
        # every run of a layer has a cache entry of its own
        schedule = tuple(RunEntry(block=i, cache=n, adds_embedding=again) for n, (i, again) in enumerate(self.run_order()))
        return ModelSpec(hidden_size=self.width, vocab_size=self.vocab, embedding_name="embed", head_name=None,
                         final_norm=self._norm("final.norm"), blocks=tuple(blocks), schedule=schedule,
                         max_positions=MAX_POSITIONS, stop_tokens=())

    def ignored_tensors(self) -> Tuple[str, ...]:
        """What a file may hold without the configuration having a use for it: the norms around a feed-forward
        that a layer does not have."""
        names = []
        for i, layer in enumerate(self.layers):
            if layer["mlp"] is None:
                names += [f"l{i}.norm2", f"l{i}.norm2b"]
        return tuple(names)

    def random_init_std(self, tensor_name: str) -> float:
        """Standard deviation for random weights: `init_std` where the configuration gives one, else
        1/sqrt(inputs) for matrices, 1 for the table's rows and 0.3 for everything else."""
        if self.init_std is not None:
            return float(self.init_std)
        if self._fan_in is None:
            from ..engine.model import expected_tensors
            self._fan_in = {n: (ts.shape[1] if len(ts.shape) == 2 else 0)
                            for n, ts in expected_tensors(self.model_spec()).items()}
        if tensor_name == "embed":
            return 1.0
        fan = self._fan_in.get(tensor_name, 0)
        return 1.0 / math.sqrt(fan) if fan else 0.3
