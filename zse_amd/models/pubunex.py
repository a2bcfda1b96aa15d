"""Pubunex: a decoder-only model whose layers are listed one by one in its config.json, some of
them run several times in a row.

A layer is a parallel layer: one RMS norm (gain stored around zero: 1 + w), and a mixer and a
feed-forward that both read it; their sum joins the residual.  The mixer is a gated delta rule
(a recurrence over a matrix state), a grouped-query attention with biases and rotary positions on
part of a head (optionally with scaled frequencies), or an attention over one cached latent row a
token with a sink per head in the softmax.  The feed-forward is a mixture of small clamped gated
layers with sigmoid scores that weigh the experts' inputs, and a shared layer on top.  Layers
``loop.start`` to ``loop.stop - 1`` run ``loop.times`` times in a row with the same weights, each
pass with a cache or state of its own; before every pass but the first the embedding's output is
added to the stream.

config.json: ``vocab``, ``width``, ``norm.eps``, ``layers`` (a list of ``{type, mixer, mlp}``),
optional ``loop`` (``start``, ``stop``, ``times``).  A ``delta`` mixer: ``heads``, ``kv_heads``, ``dim``,
``vdim``, ``conv``.  An ``attention``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, optional
``rot`` (``base``, ``dims``, optional ``scaling`` with ``factor``, ``original``, ``fast``, ``slow``).  A
``latent_attention``: ``heads``, ``dim``, ``rot_dim``, ``vdim``, ``kv_rank``, ``scale``, ``rot.base``.
``mlp``: null or ``{kind: "moe", expert: {ff, limit}, router: {experts, top}, shared: {ff, limit} or
null}``.  Tensor names: ``embed``, ``head``, ``final.norm`` and, for layer i, ``l<i>.norm1``,
``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from ..config.base import Architecture, Problems, need, register_architecture
from ..config.plan import (AttentionSpec, BlockSpec, DeltaRuleSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec,
                           LatentAttentionSpec, LayerCall, ModelPlan, NoPositionSpec, NormSpec, RotarySpec,
                           RoutedMLPSpec)

NAME = "Pubunex"
MAX_POSITION = 1 << 16        # the config names no longest sequence; tables and pools follow the runner's own limits
ACTIVATION = "clamped_swiglu"


@dataclass(frozen=True)
class PubunexMLP:
    ff: int
    limit: float
    experts: int
    top: int
    shared_ff: Optional[int]
    shared_limit: float = 0.0


@dataclass(frozen=True)
class PubunexLayer:
    type: str                          # "delta" | "attention" | "latent_attention"
    heads: int
    dim: int
    vdim: int
    mlp: Optional[PubunexMLP]
    kv_heads: int = 0
    conv: int = 0                      # delta
    scale: float = 1.0                 # both attentions
    rot_base: Optional[float] = None
    rot_dims: int = 0
    rot_scaling: Optional[Tuple[float, float, float, float]] = None
    rot_dim: int = 0                   # latent attention: the rotated part of a head
    kv_rank: int = 0


@dataclass(frozen=True)
class PubunexConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[PubunexLayer, ...]
    loop: Optional[Tuple[int, int, int]]       # start, stop, times
    raw: dict

    @staticmethod
    def _mlp(mlp: dict, q: Problems) -> Optional[PubunexMLP]:
        kind = need(mlp, "kind", str, q, default="moe")
        q.require(kind == "moe", f"mlp.kind must be 'moe', got {kind!r}")
        ex = need(mlp, "expert", dict, q, required=True) or {}
        ro = need(mlp, "router", dict, q, required=True) or {}
        sh = need(mlp, "shared", dict, q, default=None, allow_none=True)
        ff = need(ex, "ff", int, q, required=True)
        limit = need(ex, "limit", float, q, required=True)
        experts = need(ro, "experts", int, q, required=True)
        top = need(ro, "top", int, q, required=True)
        sff = need(sh, "ff", int, q, required=True) if sh is not None else None
        slim = need(sh, "limit", float, q, required=True) if sh is not None else 0.0
        if q.items:
            return None
        q.require(ff > 0 and limit > 0, f"mlp.expert: ff and limit must be positive, got {ff} and {limit}")
        q.require(1 <= top <= experts, f"mlp.router: top must lie in 1..experts, got {top} of {experts}")
        q.require(sh is None or (sff > 0 and slim > 0), f"mlp.shared: ff and limit must be positive, got {sff} and {slim}")
        return PubunexMLP(ff, limit, experts, top, sff, slim or 0.0)

    @staticmethod
    def from_dict(raw: dict) -> "PubunexConfig":
        p = Problems("Pubunex config.json")
        V = need(raw, "vocab", int, p, required=True)
        W = need(raw, "width", int, p, required=True)
        norm = need(raw, "norm", dict, p, required=True) or {}
        eps = need(norm, "eps", float, p, required=True)
        layers_raw = need(raw, "layers", list, p, required=True) or []
        loop_raw = need(raw, "loop", dict, p, default=None, allow_none=True)
        p.raise_if_any()
        p.require(V > 0 and W > 0, f"'vocab' and 'width' must be positive, got {V} and {W}")
        p.require(eps > 0, f"'norm.eps' must be positive, got {eps}")
        p.require(len(layers_raw) > 0, "'layers' is empty")
        loop = None
        if loop_raw is not None:
            start = need(loop_raw, "start", int, p, required=True)
            stop = need(loop_raw, "stop", int, p, required=True)
            times = need(loop_raw, "times", int, p, required=True)
            if None not in (start, stop, times):
                p.require(0 <= start < stop <= len(layers_raw) and times >= 1,
                          f"'loop' must name layers start < stop within the model and times >= 1, got {start}, {stop}, {times}")
                loop = (start, stop, times)
        layers = []
        for i, lr in enumerate(layers_raw):
            q = Problems(f"layer {i}")
            if not isinstance(lr, dict):
                p.add(f"layer {i} must be an object")
                continue
            typ = need(lr, "type", str, q, required=True)
            mx = need(lr, "mixer", dict, q, required=True) or {}
            mlp_raw = need(lr, "mlp", dict, q, default=None, allow_none=True)
            mlp = PubunexConfig._mlp(mlp_raw, q) if mlp_raw is not None else None
            heads = need(mx, "heads", int, q, required=True)
            dim = need(mx, "dim", int, q, required=True)
            vdim = need(mx, "vdim", int, q, required=True)
            if q.items:
                p.add(f"layer {i}: " + "; ".join(q.items))
                continue
            q.require(heads > 0 and dim > 0 and vdim > 0, "heads, dim and vdim must be positive")
            if typ == "delta":
                kvh = need(mx, "kv_heads", int, q, default=heads)
                taps = need(mx, "conv", int, q, required=True)
                if not q.items:
                    q.require(kvh > 0 and heads % kvh == 0, f"heads ({heads}) must be a multiple of kv_heads ({kvh})")
                    q.require(taps >= 1, f"conv must be at least 1, got {taps}")
                    q.require(dim <= 256 and vdim <= 1024, f"a delta layer takes dim up to 256 and vdim up to 1024, got {dim} and {vdim}")
                layers.append(PubunexLayer("delta", heads, dim, vdim, mlp, kv_heads=kvh or heads, conv=taps or 1))
            elif typ == "attention":
                kvh = need(mx, "kv_heads", int, q, default=heads)
                scale = need(mx, "scale", float, q, required=True)
                rot = need(mx, "rot", dict, q, default=None, allow_none=True)
                base = need(rot, "base", float, q, required=True) if rot is not None else None
                dims = need(rot, "dims", int, q, default=dim) if rot is not None else 0
                sc = need(rot, "scaling", dict, q, default=None, allow_none=True) if rot is not None else None
                scaling = None
                if sc is not None:
                    vals = [need(sc, key, float, q, required=True) for key in ("factor", "original", "fast", "slow")]
                    if None not in vals:
                        q.require(all(v > 0 for v in vals), f"rot.scaling: every number must be positive, got {vals}")
                        scaling = tuple(vals)
                if not q.items:
                    q.require(kvh > 0 and heads % kvh == 0, f"heads ({heads}) must be a multiple of kv_heads ({kvh})")
                    q.require(rot is None or (base > 0 and base != 1 and dims % 2 == 0 and 0 < dims <= dim),
                              f"rot.base must be positive and rot.dims even and in (0, dim], got {base} and {dims}")
                    q.require(dim <= 256 and vdim <= 256, f"an attention layer takes dim and vdim up to 256, got {dim} and {vdim}")
                layers.append(PubunexLayer("attention", heads, dim, vdim, mlp, kv_heads=kvh or heads, scale=scale or 1.0,
                                           rot_base=base, rot_dims=dims or 0, rot_scaling=scaling))
            elif typ == "latent_attention":
                scale = need(mx, "scale", float, q, required=True)
                rdim = need(mx, "rot_dim", int, q, required=True)
                rank = need(mx, "kv_rank", int, q, required=True)
                rot = need(mx, "rot", dict, q, required=True) or {}
                base = need(rot, "base", float, q, required=True)
                if not q.items:
                    q.require(rdim > 0 and rdim % 2 == 0 and rank > 0, f"rot_dim must be even and positive and kv_rank positive, got {rdim} and {rank}")
                    q.require(base > 0 and base != 1, f"rot.base must be positive, got {base}")
                    q.require(rank + rdim <= 1024, f"kv_rank + rot_dim up to 1024, got {rank + rdim}")
                layers.append(PubunexLayer("latent_attention", heads, dim, vdim, mlp, scale=scale or 1.0, rot_base=base,
                                           rot_dim=rdim or 0, kv_rank=rank or 0))
            else:
                q.add(f"unknown type {typ!r} (delta, attention, latent_attention)")
            if q.items:
                p.add(f"layer {i}: " + "; ".join(q.items))
        p.raise_if_any()
        return PubunexConfig(V, W, eps, tuple(layers), loop, dict(raw))

    def to_dict(self) -> dict:
        return dict(self.raw)

    def calls(self):
        """[(layer, the embedding is added first)] in the order the layers run."""
        n = len(self.layers)
        if self.loop is None or self.loop[2] <= 1:
            return [(i, False) for i in range(n)]
        start, stop, times = self.loop
        out = [(i, False) for i in range(start)]
        for again in range(times):
            out += [(i, again > 0 and i == start) for i in range(start, stop)]
        return out + [(i, False) for i in range(stop, n)]


def pubunex_plan(c: PubunexConfig) -> ModelPlan:
    layers = []
    for i, l in enumerate(c.layers):
        pre = f"l{i}."
        mix = pre + "mix."
        if l.type == "delta":
            mixer = DeltaRuleSpec(
                hidden_size=c.width, num_heads=l.heads, num_kv_heads=l.kv_heads, key_dim=l.dim, value_dim=l.vdim,
                conv_taps=l.conv, eps=c.eps,
                names={"q": mix + "q", "k": mix + "k", "v": mix + "v", "q_conv": mix + "q.conv", "k_conv": mix + "k.conv",
                       "v_conv": mix + "v.conv", "b": mix + "b", "a": mix + "a", "A_log": mix + "A_log",
                       "dt_bias": mix + "dt_bias", "norm": mix + "norm", "gate": mix + "g", "o": mix + "o"})
        elif l.type == "attention":
            rotary = (RotarySpec(head_dim=l.dim, rotary_dim=l.rot_dims, theta=l.rot_base, scaling=l.rot_scaling)
                      if l.rot_base is not None else NoPositionSpec())
            mixer = AttentionSpec(
                hidden_size=c.width, num_heads=l.heads, num_kv_heads=l.kv_heads, head_dim=l.dim, scale=l.scale,
                softcap=None, window=None, position=rotary,
                names={r: mix + r for r in ("q", "k", "v", "o")}, value_dim=l.vdim,
                biases={r: f"{mix}{r}.b" for r in ("q", "k", "v", "o")})
        else:
            mixer = LatentAttentionSpec(
                hidden_size=c.width, num_heads=l.heads, head_dim=l.dim, rotary_dim=l.rot_dim, value_dim=l.vdim,
                latent_dim=l.kv_rank, scale=l.scale, eps=c.eps,
                position=RotarySpec(head_dim=l.rot_dim, rotary_dim=l.rot_dim, theta=l.rot_base, interleaved=True),
                names={"q": mix + "q", "down": mix + "dkv", "down_norm": mix + "dkv.norm", "up_k": mix + "uk",
                       "up_v": mix + "uv", "o": mix + "o", "sinks": mix + "sink"})
        ffn = None
        if l.mlp is not None:
            m, mlp = l.mlp, pre + "mlp."
            shared = None
            if m.shared_ff is not None:
                shared = GatedMLPSpec(hidden_size=c.width, intermediate_size=m.shared_ff, activation=ACTIVATION,
                                      names={r: f"{mlp}shared.{r}" for r in ("gate", "up", "down")}, limit=m.shared_limit)
            ffn = RoutedMLPSpec(hidden_size=c.width, intermediate_size=m.ff, num_experts=m.experts, top_k=m.top,
                                activation=ACTIVATION, limit=m.limit, router=mlp + "router",
                                expert_names=mlp + "e{e}.{role}", shared=shared, scale_input=True)
        layers.append(BlockSpec(arrangement="parallel", mixer=mixer, ffn=ffn,
                                norms={"pre_mixer": NormSpec(c.width, c.eps, True, pre + "norm1")}))
    order = tuple(LayerCall(i, add_embedding=again) for i, again in c.calls())
    return ModelPlan(
        architecture=NAME, hidden_size=c.width, vocab_size=c.vocab, max_position=MAX_POSITION,
        embedding=EmbeddingSpec(c.vocab, c.width, 1.0, "embed"),
        layers=tuple(layers), order=order,
        final_norm=NormSpec(c.width, c.eps, True, "final.norm"),
        head=HeadSpec(c.vocab, c.width, None, "head"),
        optional_prefixes=())


PUBUNEX = register_architecture(Architecture(
    name=NAME, config_from_dict=PubunexConfig.from_dict, plan=pubunex_plan, model_types=("pubunex",)))
