"""Typed configuration of the Mimitar decoder, read from its own config.json keys.

A Mimitar model carries `streams` copies of the residual stream.  Each half of a layer reads a weighted sum of the copies through a
norm whose weights are stored around zero, and writes its result, times `residual_mult`, back into every copy with a weight of
its own while a small matrix mixes the copies (`l<i>.hc1.*` for the mixer, `l<i>.hc2.*` for the feed-forward).  The mixer's input
is first blended with the input of the token before (`l<i>.shift`).  The mixer is
  attention          grouped-query attention with one norm over the whole query projection and one over the whole key projection, a
                     rotation of the first channels of every head (half-split pairs) whose frequencies may be stretched by wavelength,
                     a scale of its own and scores capped by cap * tanh(s / cap);
  latent_attention   attention through low-rank latents with one rotated key part for all heads (neighbouring pairs, frequencies that
                     may be blended by a ramp with cosines and sines lengthened) and a gate per head on the output.
The feed-forward is a gated one with clamped halves, or a mixture of such experts behind a softmax router that may choose among the
best groups of experts only, with a gated shared expert; or absent.  A layer may run with another layer's weights and a cache of
its own (`weights_of`).  The logits are multiplied by `logit_scale`.

config.json:
    architecture  "Mimitar"
    vocab, width  sizes of the token table
    norm          {eps}: every RMS norm of the model
    streams       copies of the residual stream (default 1)
    residual_mult what a half's result is multiplied by on its way into the stream (default 1)
    logit_scale   (default 1)
    layers        [{type: "attention" | "latent_attention", mixer: {...}, mlp: null | {...}, weights_of: j (optional)}]
      attention mixer         {heads, kv_heads, dim, vdim, scale, softcap, rot: {dims, base, scaling: {factor, low, high, original}}}
      latent_attention mixer  {heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot: {dims, base, scaling: {factor, original, fast, slow}}}
                              (softcap, rot and rot.scaling may be absent or null)
      mlp                     {kind: "dense", ff, limit}
                              {kind: "moe", expert: {ff, limit}, router: {experts, top, groups: {count, keep}}, shared: {ff, limit}}
                              (groups and shared may be absent or null)
    max_positions optional: the longest sequence (default 131072)
Tensors: embed, final.norm, head, and per layer i with weights of its own under "l<i>.": norm1, norm2, shift, hc1.{in,out,mix},
hc2.{in,out,mix}, mix.*, mlp.*.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, replace
from typing import Optional, Tuple

from .errors import ConfigError
from .fekorax import _int, _number
from .registry import register_architecture
from .spec import (AttentionSpec, InterleavedRotarySpec, LatentAttentionSpec, LayerSpec, ModelSpec, PartialRotarySpec, RmsNormSpec, RotarySpec,
                   RoutedExpertsSpec, RunEntry, ScaleSpec, StreamAccessSpec, SwiGluSpec, TokenShiftSpec)

SWISH_SLOPE_ACTIVATION = "swish_clamped"      # g sigmoid(1.702 g) (u + 1) on clamped halves: the one activation of this design
RENORMALIZE_FLOOR = 1e-20                     # added to the sum the chosen experts' scores are divided by


@dataclass(frozen=True)
class WavelengthScaling:
    """Frequencies whose waves are shorter than original/high stay, those longer than original/low are divided by `factor`, and
    between the two they are blended."""
    factor: float
    low: float
    high: float
    original: int


@dataclass(frozen=True)
class RampScaling:
    """Frequencies blended between plain ones (pairs that turn fast) and ones divided by `factor` (pairs that turn slowly) by a ramp
    over the pair's index; cosines and sines are multiplied by 0.1 ln(factor) + 1."""
    factor: float
    original: int
    fast: float
    slow: float

    def magnitude(self) -> float:
        return 0.1 * math.log(self.factor) + 1.0


def wavelength_frequencies(dims: int, base: float, scaling: Optional[WavelengthScaling]):
    """The dims/2 frequencies f_i = base^(-2i/dims), stretched by the rule above where a scaling is given."""
    out = []
    for i in range(dims // 2):
        f = math.pow(float(base), -2.0 * i / dims)
        if scaling is not None:
            wave = 2.0 * math.pi / f
            if wave > scaling.original / scaling.low:
                f = f / scaling.factor
            elif not wave < scaling.original / scaling.high:
                s = (scaling.original / wave - scaling.low) / (scaling.high - scaling.low)
                f = (1.0 - s) * f / scaling.factor + s * f
        out.append(f)
    return tuple(out)


def ramp_frequencies(dims: int, base: float, scaling: Optional[RampScaling]):
    """The dims/2 frequencies.  With index(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(index(fast)), 0) and
    hi = min(ceil(index(slow)), dims - 1), pair i has the share r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1) of the slowed
    frequency: f_i / factor * r_i + f_i (1 - r_i)."""
    plain = [math.pow(float(base), -2.0 * i / dims) for i in range(dims // 2)]
    if scaling is None:
        return tuple(plain)
    index = lambda turns: dims * math.log(scaling.original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo, hi = max(math.floor(index(scaling.fast)), 0), min(math.ceil(index(scaling.slow)), dims - 1)
    out = []
    for i, f in enumerate(plain):
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f / scaling.factor * r + f * (1.0 - r))
    return tuple(out)


@dataclass(frozen=True)
class MimitarRotation:
    dims: int
    base: float
    scaling: object = None               # WavelengthScaling (attention), RampScaling (latent attention) or None


@dataclass(frozen=True)
class MimitarAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: Optional[float] = None
    rot: Optional[MimitarRotation] = None


@dataclass(frozen=True)
class MimitarLatentAttention:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: MimitarRotation = None


@dataclass(frozen=True)
class MimitarDense:
    ff: int
    limit: float


@dataclass(frozen=True)
class MimitarMoe:
    experts: int
    top: int
    ff: int
    limit: float
    groups: int = 1
    groups_kept: int = 1
    shared: Optional[MimitarDense] = None


@dataclass(frozen=True)
class MimitarLayer:
    mixer: object                        # MimitarAttention or MimitarLatentAttention
    mlp: object = None                   # MimitarDense, MimitarMoe or None
    weights_of: Optional[int] = None     # the layer whose tensors this one uses; None: its own


@dataclass(frozen=True)
class MimitarConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[MimitarLayer, ...]
    streams: int = 1
    residual_mult: float = 1.0
    logit_scale: float = 1.0
    max_positions: int = 131072
    token_shift: bool = True             # what a model folder may lack (found by the names of its tensors, `fit_to_tensors`)
    stream_weights: bool = True
    architecture: str = "Mimitar"

    # ------------------------------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, cfg: dict) -> "MimitarConfig":
        if not isinstance(cfg.get("layers"), list) or not cfg["layers"]:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(cfg["layers"]):
            where = f"layer {i}"
            if not isinstance(entry, dict) or not isinstance(entry.get("mixer"), dict):
                raise ConfigError(f"config.json: {where} needs a 'type' and a 'mixer'")
            kind = entry.get("type")
            if kind == "attention":
                mixer = cls._attention(entry["mixer"], where)
            elif kind == "latent_attention":
                mixer = cls._latent(entry["mixer"], where)
            else:
                raise ConfigError(f"config.json: {where} has the unknown type {kind!r} (attention or latent_attention)")
            weights_of = entry.get("weights_of")
            if weights_of is not None:
                weights_of = _int(entry, "weights_of", where, least=0)
            layers.append(MimitarLayer(mixer, cls._mlp(entry.get("mlp"), where), weights_of))
        for i, layer in enumerate(layers):
            if layer.weights_of is not None:
                j = layer.weights_of
                if not 0 <= j < len(layers) or j == i or layers[j].weights_of is not None:
                    raise ConfigError(f"config.json: layer {i} uses the weights of layer {j}, which must be another layer with weights of its own")
                if (type(layers[j].mixer), type(layers[j].mlp)) != (type(layer.mixer), type(layer.mlp)):
                    raise ConfigError(f"config.json: layer {i} uses the weights of layer {j} but is another kind of layer")
                layers[i] = MimitarLayer(layers[j].mixer, layers[j].mlp, j)          # (it runs as the layer whose weights it uses)
        optional = lambda key, default, **kw: default if cfg.get(key) is None else _number(cfg, key, "the model", **kw)
        return cls(vocab=_int(cfg, "vocab", "the model"), width=_int(cfg, "width", "the model"), norm_eps=_number(cfg.get("norm"), "eps", "'norm'"),
                   layers=tuple(layers), streams=1 if cfg.get("streams") is None else _int(cfg, "streams", "the model"),
                   residual_mult=optional("residual_mult", 1.0, positive=False), logit_scale=optional("logit_scale", 1.0, positive=False),
                   max_positions=131072 if cfg.get("max_positions") is None else _int(cfg, "max_positions", "the model"),
                   token_shift=bool(cfg.get("token_shift", True)), stream_weights=bool(cfg.get("stream_weights", True)))

    @staticmethod
    def _rotation(r, where, dim, latent: bool) -> Optional[MimitarRotation]:
        if r is None:
            return None
        if not isinstance(r, dict):
            raise ConfigError(f"config.json: {where}: 'rot' must be an object with 'dims' and 'base'")
        dims = _int(r, "dims", where + ", rot", least=2)
        if dims % 2 or dims > dim:
            raise ConfigError(f"config.json: {where}: rot.dims must be even and at most the head's channels")
        base = _number(r, "base", where + ", rot")
        if base == 1.0:
            raise ConfigError(f"config.json: {where}: rot.base must differ from 1")
        scaling = None
        if r.get("scaling") is not None:
            s, w = r["scaling"], where + ", rot.scaling"
            if latent:
                scaling = RampScaling(_number(s, "factor", w), _int(s, "original", w), _number(s, "fast", w), _number(s, "slow", w))
            else:
                scaling = WavelengthScaling(_number(s, "factor", w), _number(s, "low", w), _number(s, "high", w), _int(s, "original", w))
                if scaling.low == scaling.high:
                    raise ConfigError(f"config.json: {w}: 'low' and 'high' must differ")
        return MimitarRotation(dims, base, scaling)

    @classmethod
    def _attention(cls, m, where) -> MimitarAttention:
        heads, kv_heads, dim = _int(m, "heads", where), _int(m, "kv_heads", where), _int(m, "dim", where)
        if heads % kv_heads:
            raise ConfigError(f"config.json: {where}: 'heads' must be a multiple of 'kv_heads'")
        softcap = None if m.get("softcap") is None else _number(m, "softcap", where)
        return MimitarAttention(heads, kv_heads, dim, _int(m, "vdim", where), _number(m, "scale", where), softcap, cls._rotation(m.get("rot"), where, dim, False))

    @classmethod
    def _latent(cls, m, where) -> MimitarLatentAttention:
        rot_dim = _int(m, "rot_dim", where, least=2)
        rot = cls._rotation(m.get("rot"), where, rot_dim, True)
        if rot is None or rot.dims != rot_dim:
            raise ConfigError(f"config.json: {where} needs 'rot' with 'base' and 'dims' equal to 'rot_dim', an even number")
        return MimitarLatentAttention(_int(m, "heads", where), _int(m, "dim", where), rot_dim, _int(m, "vdim", where), _int(m, "q_rank", where),
                                      _int(m, "kv_rank", where), _number(m, "scale", where), rot)

    @staticmethod
    def _mlp(f, where):
        if f is None:
            return None
        w = where + ", mlp"
        if not isinstance(f, dict) or f.get("kind") not in ("dense", "moe"):
            raise ConfigError(f"config.json: {where} has a feed-forward of an unknown kind (dense, moe, or null for none)")
        if f["kind"] == "dense":
            return MimitarDense(_int(f, "ff", w), _number(f, "limit", w))
        r, e = f.get("router"), f.get("expert")
        experts, top = _int(r, "experts", w + ", router"), _int(r, "top", w + ", router")
        groups, kept = 1, 1
        if isinstance(r, dict) and r.get("groups") is not None:
            groups, kept = _int(r["groups"], "count", w + ", router.groups"), _int(r["groups"], "keep", w + ", router.groups")
        if top > experts or experts % groups or kept > groups or top > kept * (experts // groups):
            raise ConfigError(f"config.json: {w}: {experts} experts in {groups} groups of which {kept} are kept cannot give {top} to a token")
        shared = None
        if f.get("shared") is not None:
            shared = MimitarDense(_int(f["shared"], "ff", w + ", shared"), _number(f["shared"], "limit", w + ", shared"))
        return MimitarMoe(experts, top, _int(e, "ff", w + ", expert"), _number(e, "limit", w + ", expert"), groups, kept, shared)

    def fit_to_tensors(self, names) -> "MimitarConfig":
        """The configuration of a folder whose tensors have these names: a model may come without the blend with the token before
        (no `l<i>.shift`) or, with one copy of the stream, without the copies' weights (no `l<i>.hc1.in`)."""
        names = set(names)
        own = [i for i, l in enumerate(self.layers) if l.weights_of is None]
        return replace(self, token_shift=self.token_shift and any(f"l{i}.shift" in names for i in own),
                       stream_weights=self.stream_weights and (self.streams > 1 or any(f"l{i}.hc1.in" in names for i in own)))

    def to_dict(self) -> dict:
        """config.json content that `from_dict` reads back to an equal configuration."""
        def rotation(r):
            d = dict(dims=r.dims, base=r.base)
            if isinstance(r.scaling, WavelengthScaling):
                d["scaling"] = dict(factor=r.scaling.factor, low=r.scaling.low, high=r.scaling.high, original=r.scaling.original)
            elif isinstance(r.scaling, RampScaling):
                d["scaling"] = dict(factor=r.scaling.factor, original=r.scaling.original, fast=r.scaling.fast, slow=r.scaling.slow)
            return d
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, MimitarAttention):
                mixer, kind = dict(heads=m.heads, kv_heads=m.kv_heads, dim=m.dim, vdim=m.vdim, scale=m.scale), "attention"
                if m.softcap is not None:
                    mixer["softcap"] = m.softcap
                if m.rot is not None:
                    mixer["rot"] = rotation(m.rot)
            else:
                mixer, kind = dict(heads=m.heads, dim=m.dim, rot_dim=m.rot_dim, vdim=m.vdim, q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale,
                                   rot=rotation(m.rot)), "latent_attention"
            f = layer.mlp
            if isinstance(f, MimitarDense):
                mlp = dict(kind="dense", ff=f.ff, limit=f.limit)
            elif isinstance(f, MimitarMoe):
                mlp = dict(kind="moe", expert=dict(ff=f.ff, limit=f.limit), router=dict(experts=f.experts, top=f.top))
                if f.groups > 1:
                    mlp["router"]["groups"] = dict(count=f.groups, keep=f.groups_kept)
                if f.shared is not None:
                    mlp["shared"] = dict(ff=f.shared.ff, limit=f.shared.limit)
            else:
                mlp = None
            entry = dict(type=kind, mixer=mixer, mlp=mlp)
            if layer.weights_of is not None:
                entry["weights_of"] = layer.weights_of
            layers.append(entry)
        out = dict(architecture=self.architecture, vocab=self.vocab, width=self.width, norm=dict(eps=self.norm_eps), streams=self.streams,
                   residual_mult=self.residual_mult, logit_scale=self.logit_scale, layers=layers, max_positions=self.max_positions)
        if not self.token_shift:
            out["token_shift"] = False
        if not self.stream_weights:
            out["stream_weights"] = False
        return out

    # ------------------------------------------------------------------------------------ as parts
    def _feed_forward(self, f, m):
        width = self.width
        gated = lambda p, d: SwiGluSpec(width, d.ff, p + "gate", p + "up", p + "down", activation=SWISH_SLOPE_ACTIVATION, activation_limit=d.limit)
        if f is None:
            return None
        if isinstance(f, MimitarDense):
            return gated(m, f)
        e = range(f.experts)
        return RoutedExpertsSpec(hidden_size=width, intermediate_size=f.ff, n_experts=f.experts, top=f.top, router=m + "router",
                                 gate_projs=tuple(f"{m}e{j}.gate" for j in e), up_projs=tuple(f"{m}e{j}.up" for j in e), down_projs=tuple(f"{m}e{j}.down" for j in e),
                                 score="softmax", renormalize=True, weigh="output", activation=SWISH_SLOPE_ACTIVATION, activation_limit=f.limit,
                                 shared=None if f.shared is None else gated(m + "shared.", f.shared), shared_gate=None if f.shared is None else m + "shared.sg",
                                 n_groups=f.groups, groups_kept=f.groups_kept, renormalize_floor=RENORMALIZE_FLOOR)

    def model_spec(self) -> ModelSpec:
        eps, width = self.norm_eps, self.width
        if self.streams > 1 and not self.stream_weights:
            raise ConfigError("a model with several copies of the residual stream needs the weights that read and write them")
        specs, index_of = [], {}
        for i, layer in enumerate(self.layers):
            if layer.weights_of is not None:
                continue
            p, m = f"l{i}.", layer.mixer
            x = p + "mix."
            if isinstance(m, MimitarAttention):
                position = None
                if m.rot is not None:
                    frequencies = wavelength_frequencies(m.rot.dims, m.rot.base, m.rot.scaling)
                    position = RotarySpec(m.dim, m.rot.base, frequencies) if m.rot.dims == m.dim else PartialRotarySpec(m.dim, m.rot.dims, m.rot.base, frequencies)
                mixer = AttentionSpec(hidden_size=width, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim, q_proj=x + "q", k_proj=x + "k", v_proj=x + "v",
                                      o_proj=x + "o", position=position, value_dim=m.vdim, scale=m.scale, q_norm=x + "q.norm", k_norm=x + "k.norm",
                                      qk_norm_eps=eps, qk_norm_whole=True, score_cap=m.softcap)
            else:
                magnitude = m.rot.scaling.magnitude() if m.rot.scaling is not None else 1.0
                mixer = LatentAttentionSpec(hidden_size=width, n_heads=m.heads, head_dim=m.dim, rotary_dim=m.rot_dim, value_dim=m.vdim, q_rank=m.q_rank,
                                            kv_rank=m.kv_rank, scale=m.scale, norm_eps=eps, dq_proj=x + "dq", dq_norm=x + "dq.norm", uq_proj=x + "uq",
                                            dkv_proj=x + "dkv", dkv_norm=x + "dkv.norm", uk_proj=x + "uk", uv_proj=x + "uv", o_proj=x + "o",
                                            position=InterleavedRotarySpec(m.rot_dim, m.rot.base, ramp_frequencies(m.rot_dim, m.rot.base, m.rot.scaling), magnitude),
                                            head_gate=x + "g")
            if self.token_shift:
                mixer = TokenShiftSpec(width, p + "shift", mixer)
            access = lambda q: StreamAccessSpec(self.streams, f"{p}hc{q}.in", f"{p}hc{q}.out", f"{p}hc{q}.mix") if self.stream_weights else None
            ff = self._feed_forward(layer.mlp, p + "mlp.")
            index_of[i] = len(specs)
            specs.append(LayerSpec(mixer=mixer, feed_forward=ff, mixer_norm=RmsNormSpec(width, eps, p + "norm1", weight_offset=1.0),
                                   feed_forward_norm=None if ff is None else RmsNormSpec(width, eps, p + "norm2", weight_offset=1.0), block="multistream",
                                   mixer_streams=access(1), feed_forward_streams=None if ff is None else access(2), residual_scale=self.residual_mult))
        unused = tuple(rf"l{i}\.(norm2|hc2\.(in|out|mix))" for i, l in enumerate(self.layers) if l.weights_of is None and l.mlp is None)      # a layer without a feed-forward reads none of them
        run_order = tuple(RunEntry(index_of[i if l.weights_of is None else l.weights_of]) for i, l in enumerate(self.layers))
        return ModelSpec(architecture=self.architecture, vocab_size=self.vocab, hidden_size=width, max_positions=self.max_positions, embedding="embed",
                         final_norm=RmsNormSpec(width, eps, "final.norm", weight_offset=1.0), lm_head="head", layers=tuple(specs), run_order=run_order,
                         ignorable_tensors=unused, after_head=() if self.logit_scale == 1.0 else (ScaleSpec(self.logit_scale),), n_streams=self.streams)


register_architecture(MimitarConfig.architecture, MimitarConfig, model_type="mimitar")
