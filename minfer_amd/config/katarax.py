"""Katarax: a decoder whose layers read the stream through one RMS norm (gain one plus the stored weight) and add a
mixer's and a feed-forward's result side by side, x <- x + mixer(N(x)) + ff(N(x)).  A mixer is
  "attention":        grouped-query softmax attention without rotation, with a learned number per (bucket of the
                      distance, head) added to the scaled score, a sliding window and the sequence's first
                      positions kept in sight;
  "latent_attention": attention over one normed latent a token and one rotated key part all heads share, queries
                      through a normed latent of their own, rotation in neighbouring pairs, a sliding window, the
                      heads' results times sigmoid(Wg x) value by value;
  "attention_2":      grouped-query causal attention with a rotation in halves and queries and keys over their root
                      mean square per head; a layer with `kv_from` has no key and value matrices and reads the keys
                      and values of the layer it names.
A feed-forward is a mixture of clamped gated experts; its router scores with a sigmoid, chooses by score plus a
correction per expert among the experts of the best groups (a group counts the sum of its two best), and weighs by
the scores over their sum, times a scale.  The logits may be capped by cap tanh(z / cap).

config.json: `architecture` = "Katarax"; `vocab`, `width`; `norm` = {eps}; `logit_softcap` or absent; `layers`, a
list of {type, mixer: {...}, mlp: {...} or null}.
Mixer sizes: attention {heads, kv_heads, dim, vdim, scale, bias_max, mask: {size, keep_first}};
latent_attention {heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rot: {base, dims}, mask: {size}};
attention_2 {heads, kv_heads, dim, vdim, scale, rot: {base, dims}, kv_from}.
mlp: {kind: "moe", expert: {ff, limit}, router: {experts, top, scale, groups: {count, keep}}}.
The rows of an attention layer's bias table are the first size of its tensor `l<i>.mix.rel` (`bias_rows` in a
configuration that is written without a file).
Tensors: embed, l<i>.norm1, l<i>.mix.*, l<i>.mlp.*, final.norm, head.
"""
from __future__ import annotations

import copy
import math
from typing import Any, Dict, List, Mapping, Optional, Sequence, Tuple

from .base import ConfigError, KeyReader
from ..parts.spec import BlockSpec, ModelSpec, PartSpec, RunEntry

ARCHITECTURE = "Katarax"
MIXER_TYPES = ("attention", "latent_attention", "attention_2")
MAX_POSITIONS = 1 << 20      # the design names no bound; rotation tables grow on demand up to here
GROUP_TOP = 2                # a group of experts counts the sum of its two best corrected scores


def _mask(raw: Any, where: str, keeps: bool) -> Optional[Dict[str, int]]:
    if raw is None:
        return None
    k = KeyReader(raw, where)
    out = dict(size=k.integer("size"))
    if keeps:
        out["keep_first"] = k.integer("keep_first", default=0, minimum=0)
    return out


def _rotation(raw: Any, where: str, most: int) -> Dict[str, Any]:
    k = KeyReader(raw or {}, where)
    dims = k.integer("dims")
    if dims % 2 or dims > most:
        raise ConfigError(f"{where}: 'dims' must be even and at most {most}, found {dims}")
    return dict(base=k.number("base"), dims=dims)


def _mixer_sizes(kind: str, raw: Any, where: str) -> Dict[str, Any]:
    r = KeyReader(raw, where)
    if kind == "latent_attention":
        out = dict(heads=r.integer("heads"), dim=r.integer("dim"), rot_dim=r.integer("rot_dim"), vdim=r.integer("vdim"),
                   kv_rank=r.integer("kv_rank"), q_rank=r.integer("q_rank"), scale=r.number("scale"))
        out["rot"] = _rotation(r.raw_value("rot"), where + ".rot", out["rot_dim"])
        out["mask"] = _mask(r.raw_value("mask"), where + ".mask", keeps=False)
        return out
    out = dict(heads=r.integer("heads"), kv_heads=r.integer("kv_heads"), dim=r.integer("dim"), vdim=r.integer("vdim"),
               scale=r.number("scale"))
    if out["heads"] % out["kv_heads"]:
        raise ConfigError(f"{where}: 'heads' {out['heads']} is not a multiple of 'kv_heads' {out['kv_heads']}")
    if kind == "attention":
        out["bias_max"] = r.number("bias_max")
        out["bias_rows"] = r.integer("bias_rows", default=None, minimum=2)
        out["mask"] = _mask(r.raw_value("mask"), where + ".mask", keeps=True)
        return out
    out["rot"] = _rotation(r.raw_value("rot"), where + ".rot", out["dim"])
    out["kv_from"] = r.integer("kv_from", default=None, minimum=0)
    return out


def _mlp_sizes(raw: Any, where: str) -> Optional[Dict[str, Any]]:
    if raw is None:
        return None
    m = KeyReader(raw, where)
    kind = m.string("kind", default="moe")
    if kind != "moe":
        raise ConfigError(f"{where}: kind {kind!r} is not one of ['moe']")
    e = KeyReader(m.raw_value("expert") or {}, where + ".expert")
    r = KeyReader(m.raw_value("router") or {}, where + ".router")
    g = KeyReader(r.raw_value("groups") or {}, where + ".router.groups")
    count = g.integer("count", default=1)
    out = dict(kind="moe", expert=dict(ff=e.integer("ff"), limit=e.number("limit")),
               router=dict(experts=r.integer("experts"), top=r.integer("top"), scale=r.number("scale", default=1.0),
                           groups=dict(count=count, keep=g.integer("keep", default=count))))
    rt = out["router"]
    if rt["experts"] % count or not 1 <= rt["groups"]["keep"] <= count:
        raise ConfigError(f"{where}.router.groups: {rt['experts']} experts do not form {count} equal groups of which "
                          f"{rt['groups']['keep']} are kept")
    if rt["top"] > rt["groups"]["keep"] * (rt["experts"] // count):
        raise ConfigError(f"{where}.router: {rt['top']} experts cannot be chosen from {rt['groups']['keep']} groups of "
                          f"{rt['experts'] // count}")
    return out


class KataraxConfig:
    architecture = ARCHITECTURE

    def __init__(self, vocab: int, width: int, eps: float, layers: List[Dict[str, Any]],
                 logit_softcap: Optional[float] = None, init_std: Optional[float] = None):
        self.vocab, self.width, self.eps = vocab, width, eps
        self.layers, self.logit_softcap = layers, logit_softcap
        self.init_std = init_std
        self._fan_in: Optional[Dict[str, int]] = None

    # ---------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "KataraxConfig":
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
        for i, layer in enumerate(layers):
            j = layer["mixer"].get("kv_from")
            if j is None:
                continue
            where = f"config.json: layers[{i}].mixer"
            if j >= i or layers[j]["type"] != "attention_2" or layers[j]["mixer"].get("kv_from") is not None:
                raise ConfigError(f"{where}: 'kv_from' {j} must name an earlier attention_2 layer with keys and values "
                                  "of its own")
            mine, theirs = layer["mixer"], layers[j]["mixer"]
            for key in ("heads", "kv_heads", "dim", "vdim", "rot"):
                if mine[key] != theirs[key]:
                    raise ConfigError(f"{where}: '{key}' {mine[key]} differs from that of layer {j} ({theirs[key]}), "
                                      "whose keys and values this layer reads")
        cap = r.raw_value("logit_softcap")
        return cls(vocab, width, eps, layers, logit_softcap=None if cap is None else r.number("logit_softcap"),
                   init_std=raw.get("init_std"))

    def adopt_tensor_shapes(self, shapes: Mapping[str, Sequence[int]]) -> None:
        """Sizes that only the tensors give: the rows of every attention layer's bias table."""
        for i, layer in enumerate(self.layers):
            if layer["type"] != "attention" or layer["mixer"].get("bias_rows") is not None:
                continue
            shape = shapes.get(f"l{i}.mix.rel")
            if shape is None or len(shape) != 2 or shape[0] < 2:
                raise ConfigError(f"config.json: layers[{i}].mixer: the bias table l{i}.mix.rel gives the number of "
                                  f"distance buckets; found shape {None if shape is None else list(shape)}")
            layer["mixer"]["bias_rows"] = int(shape[0])

    def to_dict(self) -> Dict[str, Any]:
        """A config.json that reads back to this configuration."""
        d = dict(architecture=ARCHITECTURE, vocab=self.vocab, width=self.width, norm=dict(eps=self.eps),
                 layers=copy.deepcopy(self.layers))
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        if self.init_std is not None:
            d["init_std"] = self.init_std
        return d

    # ---------------------------------------------------------------- description
    def _norm(self, name: str) -> PartSpec:
        return PartSpec("offset_rmsnorm", dict(size=self.width, eps=self.eps, weight=name))

    def _mixer(self, i: int, layer: Dict[str, Any]) -> PartSpec:
        m, kind = layer["mixer"], layer["type"]
        names = {k: "mix." + k for k in ("q", "k", "v", "o")}
        window = None if m.get("mask") is None else m["mask"]["size"]
        if kind == "latent_attention":
            rot = m["rot"]
            return PartSpec("latent_attention", dict(
                hidden_size=self.width, n_heads=m["heads"], dim=m["dim"], rot_dim=m["rot_dim"], v_dim=m["vdim"],
                rank=m["kv_rank"], q_rank=m["q_rank"], scale=m["scale"], eps=self.eps, window=window, gate_per_value=True,
                position=PartSpec("rope_pairs", dict(dims=rot["dims"], base=rot["base"], scaling=None,
                                                     max_positions=MAX_POSITIONS)),
                q="mix.uq", dq="mix.dq", dq_norm="mix.dq.norm", dkv="mix.dkv", dkv_norm="mix.dkv.norm", uk="mix.uk",
                uv="mix.uv", gate="mix.g", o="mix.o"))
        common = dict(hidden_size=self.width, n_heads=m["heads"], n_kv_heads=m["kv_heads"], dim=m["dim"], v_dim=m["vdim"],
                      scale=m["scale"], eps=self.eps, **names)
        if kind == "attention":
            if m.get("bias_rows") is None:
                raise ConfigError(f"config.json: layers[{i}].mixer: the number of distance buckets is the first size of "
                                  f"l{i}.mix.rel; without a file, give 'bias_rows'")
            if not m["bias_max"] > m["bias_rows"] // 2:
                raise ConfigError(f"config.json: layers[{i}].mixer: 'bias_max' {m['bias_max']} must lie beyond half the "
                                  f"{m['bias_rows']} buckets")
            keep = 0 if m.get("mask") is None else m["mask"].get("keep_first", 0)
            return PartSpec("normed_attention", dict(
                common, qk_norm=False, window=window, keep_first=keep or None,
                distance_bias=dict(table="mix.rel", rows=m["bias_rows"], far=m["bias_max"])))
        rot = m["rot"]
        return PartSpec("normed_attention", dict(
            common, qk_norm=True, qk_gains=False, shared_kv=m.get("kv_from") is not None,
            position=PartSpec("rope_half", dict(dims=rot["dims"], base=rot["base"], scaling=None,
                                                max_positions=MAX_POSITIONS))))

    def _feed_forward(self, mlp: Dict[str, Any]) -> PartSpec:
        r = mlp["router"]
        return PartSpec("grouped_moe", dict(
            hidden_size=self.width, intermediate_size=mlp["expert"]["ff"], n_experts=r["experts"], top=r["top"],
            groups=r["groups"]["count"], keep=r["groups"]["keep"], act="clamped_swish", limit=mlp["expert"]["limit"],
            score="sigmoid", correction="mlp.correction", group_top=GROUP_TOP, weight_scale=r["scale"],
            router="mlp.router", expert="mlp.e{}"))

    def model_spec(self) -> ModelSpec:
        blocks, schedule = [], []
        for i, layer in enumerate(self.layers):
            ffn = None if layer["mlp"] is None else self._feed_forward(layer["mlp"])
            blocks.append(BlockSpec(kind="parallel_shared_norm", prefix=f"l{i}.", mixer=self._mixer(i, layer),
                                    feed_forward=ffn, norms={"input": self._norm("norm1")}))
            # a layer that reads another layer's keys and values runs on that layer's cache entry and writes nothing
            j = layer["mixer"].get("kv_from")
            schedule.append(RunEntry(block=i, cache=i if j is None else j, writes_cache=j is None))
        sizes = dict(vocab_size=self.vocab, hidden_size=self.width, name="head")
        head = PartSpec("linear_head", sizes) if self.logit_softcap is None else \
            PartSpec("capped_linear_head", dict(sizes, cap=self.logit_softcap))
        return ModelSpec(hidden_size=self.width, vocab_size=self.vocab, embedding_name="embed", head=head,
                         final_norm=self._norm("final.norm"), blocks=tuple(blocks), schedule=tuple(schedule),
                         max_positions=MAX_POSITIONS, stop_tokens=())

    def random_init_std(self, tensor_name: str) -> float:
        """Standard deviation for random weights: `init_std` where the configuration gives one, else
        1/sqrt(inputs) for matrices, 1 for the table's rows and 0.3 for everything else."""
        if self.init_std is not None:
            return float(self.init_std)
        if self._fan_in is None:
            from ..engine.model import expected_tensors
            self._fan_in = {n: (ts.shape[1] if len(ts.shape) == 2 and not n.endswith(".rel") else 0)
                            for n, ts in expected_tensors(self.model_spec()).items()}
        if tensor_name == "embed":
            return 1.0
        fan = self._fan_in.get(tensor_name, 0)
        return 1.0 / math.sqrt(fan) if fan else 0.3
