"""Typed configuration of the Zidevik decoder, read from its own config.json keys.

A Zidevik model is a list of "parallel" layers: one norm, whose rows both the mixer and the feed-forward (if the layer has one)
read, and both results join the residual stream.  Behind that every layer takes a second, small input from the token itself (a
slice of a second token table, gated by the stream, projected, normed and added), if the model has such a table.  The mixer is
two mixers side by side on the same rows, their results added with a weight each:
  left   grouped-query attention: a rotation of the neighbouring pairs (2i, 2i + 1) of a head's first channels, then every query
         and key head divided by its root mean square; a score scale of its own; causal softmax;
  right  a selective scan (the Mamba recurrence) behind a short causal convolution.
The feed-forward is a gated one (SiLU), or a mixture of such experts: a 32-bit sigmoid router, the `top` largest scores choose,
a chosen expert's score multiplies its input (no renormalising), and a shared expert serves every row.
A run of layers may be walked several times with the same weights (`loop`): every walk keeps caches and states of its own and
is entered through a product of [stream; token rows] plus a vector per walk.  The logits are soft-capped.

config.json:
    architecture  "Zidevik"
    vocab, width  sizes of the token table
    norm          {eps}: every RMS norm of the model
    layers        [{type: "parallel", mixer: {left: {heads, kv_heads, dim, vdim, scale, rot: {dims, base}}, left_scale,
                                                  right: {inner, state, dt_rank, conv}, right_scale},
                    mlp: null | {kind: "dense", ff} | {kind: "moe", router: {experts, top}, expert: {ff}, shared: {ff}}}]
                  (rot and shared may be absent or null)
    loop          optional {start, stop, times}: layers start .. stop - 1 are walked `times` times in a row
    token_side    optional {dim}: every layer reads `dim` columns of the second token table, layer i its own
    logit_softcap optional
    max_positions optional: the longest sequence (default 131072)
Tensors: embed, final.norm, head, (loop.in, loop.step), (side.embed), and per layer i under "l<i>.": norm1, mix.left.{q,k,v,o},
mix.right.{in,conv,conv.b,x,dt,dt.b,A_log,D,o}, mlp.{gate,up,down} or mlp.{router, e<j>.{gate,up,down}, shared.{gate,up,down}},
(side.gate, side.proj, side.norm).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .errors import ConfigError
from .fekorax import _int, _number
from .registry import register_architecture
from .spec import (AttentionSpec, InterleavedRotarySpec, LayerSpec, ModelSpec, RejoinSpec, RmsNormSpec, RoutedExpertsSpec, RunEntry, SelectiveScanSpec,
                   SideBySideSpec, SoftCapSpec, SwiGluSpec, TokenSideInputSpec)


@dataclass(frozen=True)
class ZidevikAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: Optional[int] = None
    rot_base: Optional[float] = None


@dataclass(frozen=True)
class ZidevikScan:
    inner: int
    state: int
    dt_rank: int
    conv: int


@dataclass(frozen=True)
class ZidevikMlp:
    kind: str                        # "dense" or "moe"
    ff: int                          # of the dense feed-forward, or of one expert
    experts: int = 0
    top: int = 0
    shared_ff: Optional[int] = None


@dataclass(frozen=True)
class ZidevikLayer:
    left: ZidevikAttention
    left_scale: float
    right: ZidevikScan
    right_scale: float
    mlp: Optional[ZidevikMlp]


@dataclass(frozen=True)
class ZidevikLoop:
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class ZidevikConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[ZidevikLayer, ...]
    loop: Optional[ZidevikLoop] = None
    side_dim: Optional[int] = None
    logit_softcap: Optional[float] = None
    max_positions: int = 131072
    architecture: str = "Zidevik"

    @classmethod
    def from_dict(cls, cfg: dict) -> "ZidevikConfig":
        if not isinstance(cfg.get("layers"), list) or not cfg["layers"]:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(cfg["layers"]):
            where = f"layer {i}"
            if not isinstance(entry, dict) or not isinstance(entry.get("mixer"), dict):
                raise ConfigError(f"config.json: {where} needs a 'type' and a 'mixer'")
            if entry.get("type") != "parallel":
                raise ConfigError(f"config.json: {where} has the unknown type {entry.get('type')!r} (parallel)")
            m = entry["mixer"]
            l, r = m.get("left"), m.get("right")
            if not isinstance(l, dict) or not isinstance(r, dict):
                raise ConfigError(f"config.json: {where}: the mixer needs 'left' and 'right'")
            heads, kv_heads, dim = _int(l, "heads", where), _int(l, "kv_heads", where), _int(l, "dim", where)
            if heads % kv_heads:
                raise ConfigError(f"config.json: {where}: 'heads' must be a multiple of 'kv_heads'")
            rot_dims = rot_base = None
            if l.get("rot") is not None:
                rot_dims, rot_base = _int(l["rot"], "dims", where + ", rot", least=2), _number(l["rot"], "base", where + ", rot")
                if rot_dims % 2 or rot_dims > dim:
                    raise ConfigError(f"config.json: {where}: rot.dims must be even and at most 'dim'")
            left = ZidevikAttention(heads, kv_heads, dim, _int(l, "vdim", where), _number(l, "scale", where), rot_dims, rot_base)
            right = ZidevikScan(_int(r, "inner", where), _int(r, "state", where), _int(r, "dt_rank", where), _int(r, "conv", where))
            mlp = entry.get("mlp")
            if mlp is not None:
                w = where + ", mlp"
                if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
                    raise ConfigError(f"config.json: {where} has a feed-forward of an unknown kind (dense, moe, or null for none)")
                if mlp["kind"] == "dense":
                    mlp = ZidevikMlp("dense", _int(mlp, "ff", w))
                else:
                    router, shared = mlp.get("router"), mlp.get("shared")
                    experts, top = _int(router, "experts", w + ", router"), _int(router, "top", w + ", router")
                    if top > experts:
                        raise ConfigError(f"config.json: {w}: 'top' cannot exceed 'experts'")
                    mlp = ZidevikMlp("moe", _int(mlp.get("expert"), "ff", w + ", expert"), experts, top, None if shared is None else _int(shared, "ff", w + ", shared"))
            layers.append(ZidevikLayer(left, _number(m, "left_scale", where, positive=False), right, _number(m, "right_scale", where, positive=False), mlp))
        loop = None
        if cfg.get("loop") is not None:
            lp = cfg["loop"]
            loop = ZidevikLoop(_int(lp, "start", "'loop'", least=0), _int(lp, "stop", "'loop'", least=0), _int(lp, "times", "'loop'", least=1))
            if not loop.start <= loop.stop <= len(layers):
                raise ConfigError("config.json: 'loop' needs 0 <= start <= stop <= the number of layers")
        side, cap, max_positions = cfg.get("token_side"), cfg.get("logit_softcap"), cfg.get("max_positions")
        return cls(vocab=_int(cfg, "vocab", "the model"), width=_int(cfg, "width", "the model"), norm_eps=_number(cfg.get("norm"), "eps", "'norm'"),
                   layers=tuple(layers), loop=loop, side_dim=None if side is None else _int(side, "dim", "'token_side'"),
                   logit_softcap=None if cap is None else _number(cfg, "logit_softcap", "the model"),
                   max_positions=131072 if max_positions is None else _int(cfg, "max_positions", "the model"))

    def to_dict(self) -> dict:
        """config.json content that `from_dict` reads back to an equal configuration."""
        layers = []
        for layer in self.layers:
            a, r = layer.left, layer.right
            left = dict(heads=a.heads, kv_heads=a.kv_heads, dim=a.dim, vdim=a.vdim, scale=a.scale)
            if a.rot_dims is not None:
                left["rot"] = dict(dims=a.rot_dims, base=a.rot_base)
            mixer = dict(left=left, left_scale=layer.left_scale, right=dict(inner=r.inner, state=r.state, dt_rank=r.dt_rank, conv=r.conv), right_scale=layer.right_scale)
            mlp = layer.mlp
            if mlp is not None and mlp.kind == "dense":
                mlp = dict(kind="dense", ff=mlp.ff)
            elif mlp is not None:
                d = dict(kind="moe", router=dict(experts=mlp.experts, top=mlp.top), expert=dict(ff=mlp.ff))
                if mlp.shared_ff is not None:
                    d["shared"] = dict(ff=mlp.shared_ff)
                mlp = d
            layers.append(dict(type="parallel", mixer=mixer, mlp=mlp))
        out = dict(architecture=self.architecture, vocab=self.vocab, width=self.width, norm=dict(eps=self.norm_eps), layers=layers, max_positions=self.max_positions)
        if self.loop is not None:
            out["loop"] = dict(start=self.loop.start, stop=self.loop.stop, times=self.loop.times)
        if self.side_dim is not None:
            out["token_side"] = dict(dim=self.side_dim)
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        return out

    # ------------------------------------------------------------------------------------ as parts
    def layer_order(self):
        """[(layer, number of the walk that begins with this entry, or None)] in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, None) for i in range(n)]
        lp = self.loop
        order = [(i, None) for i in range(lp.start)]
        for t in range(lp.times):
            order += [(i, t if i == lp.start else None) for i in range(lp.start, lp.stop)]
        return order + [(i, None) for i in range(lp.stop, n)]

    def model_spec(self) -> ModelSpec:
        eps, width = self.norm_eps, self.width
        specs = []
        for i, layer in enumerate(self.layers):
            p, a, r = f"l{i}.", layer.left, layer.right
            x = p + "mix.left."
            left = AttentionSpec(hidden_size=width, n_heads=a.heads, n_kv_heads=a.kv_heads, head_dim=a.dim, q_proj=x + "q", k_proj=x + "k", v_proj=x + "v",
                                 o_proj=x + "o", position=None if a.rot_dims is None else InterleavedRotarySpec(a.rot_dims, a.rot_base), value_dim=a.vdim,
                                 scale=a.scale, qk_unit_rms=True, qk_norm_eps=eps)
            x = p + "mix.right."
            right = SelectiveScanSpec(hidden_size=width, inner=r.inner, state=r.state, dt_rank=r.dt_rank, conv_taps=r.conv, in_proj=x + "in", conv=x + "conv",
                                      conv_bias=x + "conv.b", x_proj=x + "x", dt_proj=x + "dt", dt_bias=x + "dt.b", a_log=x + "A_log", d_skip=x + "D", o_proj=x + "o")
            mixer = SideBySideSpec(width, (left, right), (layer.left_scale, layer.right_scale))
            ff, m = None, p + "mlp."
            if layer.mlp is not None and layer.mlp.kind == "dense":
                ff = SwiGluSpec(width, layer.mlp.ff, m + "gate", m + "up", m + "down")
            elif layer.mlp is not None:
                e = range(layer.mlp.experts)
                shared = None if layer.mlp.shared_ff is None else SwiGluSpec(width, layer.mlp.shared_ff, m + "shared.gate", m + "shared.up", m + "shared.down")
                ff = RoutedExpertsSpec(hidden_size=width, intermediate_size=layer.mlp.ff, n_experts=layer.mlp.experts, top=layer.mlp.top, router=m + "router",
                                       gate_projs=tuple(f"{m}e{j}.gate" for j in e), up_projs=tuple(f"{m}e{j}.up" for j in e),
                                       down_projs=tuple(f"{m}e{j}.down" for j in e), score="sigmoid", renormalize=False, weigh="input", shared=shared)
            after = ()
            if self.side_dim is not None:
                d = self.side_dim
                after = (TokenSideInputSpec(hidden_size=width, vocab_size=self.vocab, dim=d, table="side.embed", table_width=d * len(self.layers), first_column=i * d,
                                            gate_proj=p + "side.gate", out_proj=p + "side.proj", norm=RmsNormSpec(width, eps, p + "side.norm"), activation="gelu_tanh"),)
            specs.append(LayerSpec(mixer=mixer, feed_forward=ff, mixer_norm=RmsNormSpec(width, eps, p + "norm1"), feed_forward_norm=None, block="parallel", after=after))
        times = self.loop.times if self.loop is not None else 0
        run_order = tuple(RunEntry(i, before=None if walk is None else RejoinSpec(width, "loop.in", "loop.step", times, walk)) for i, walk in self.layer_order())
        unused = ()
        if self.loop is not None and self.loop.start == self.loop.stop:          # walks without a layer: their tensors are in the file and are not read
            unused = (r"loop\.in", r"loop\.step")
        return ModelSpec(architecture=self.architecture, vocab_size=self.vocab, hidden_size=width, max_positions=self.max_positions, embedding="embed",
                         final_norm=RmsNormSpec(width, eps, "final.norm"), lm_head="head", layers=tuple(specs), run_order=run_order, ignorable_tensors=unused,
                         after_head=() if self.logit_softcap is None else (SoftCapSpec(self.logit_softcap),))


register_architecture("Zidevik", ZidevikConfig, model_type="zidevik")
