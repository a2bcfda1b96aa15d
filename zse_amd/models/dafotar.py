"""Dafotar: a decoder-only model whose layers are listed one by one in its config.json.

Every layer is a pre-norm layer over ``streams`` residual streams (layer norms with bias, a
short causal convolution between the first norm and the mixer) whose mixer is either a
sliding-window attention (a norm over each query and key head, a number per query head on
the scores, rotary positions on part of a head, values stored rotated over all their channels
and outputs turned back, keys and values possibly read from another layer) or a matrix-memory
recurrence (mLSTM); its feed-forward, where it has one, is relu(gate) * up.  The head is the
embedding table, behind a layer norm of the streams' sum.

config.json: ``vocab``, ``width``, ``norm.eps``, ``layers`` (a list of ``{type, mixer, mlp}``);
optional ``streams`` (absent: one residual, plain sums), ``canon.taps`` (absent: no
convolution).  An attention's ``mixer``: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``,
optional ``mask.size`` (absent: every earlier key is seen), ``rot.base`` / ``rot.dims`` (absent:
no rotation at all) and ``kv_from``.  An mlstm's: ``heads``, ``dim``, ``vdim``, ``gate_cap``.
``mlp``: null or ``{kind: "dense", ff}``.  Tensor names: ``embed``, ``final.norm[.b]`` and, for
layer i, ``l<i>.norm<q>[.b]``, ``l<i>.canon1``, ``l<i>.hc<q>.{in,out,mix}``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from ..config.base import Architecture, Problems, need, register_architecture
from ..config.plan import (AttentionSpec, EmbeddingSpec, GatedMLPSpec, HeadSpec, LayerCall, LayerNormSpec,
                           MatrixMemorySpec, ModelPlan, NoPositionSpec, RotarySpec, ShortConvSpec,
                           StreamsBlockSpec)

NAME = "Dafotar"
MAX_POSITION = 1 << 16        # the config names no longest sequence: the longest the engine's decode attention takes for any head size;
#                               tables and pools are sized by the runner's own limits


@dataclass(frozen=True)
class DafotarLayer:
    type: str                          # "attention" | "mlstm"
    heads: int
    dim: int
    vdim: int
    ff: Optional[int]                  # None: no feed-forward
    # attention
    kv_heads: int = 0
    scale: float = 1.0
    window: Optional[int] = None
    rot_base: Optional[float] = None
    rot_dims: int = 0
    kv_from: Optional[int] = None
    # mlstm
    gate_cap: float = 0.0


@dataclass(frozen=True)
class DafotarConfig:
    vocab: int
    width: int
    eps: float
    streams: Optional[int]
    taps: Optional[int]
    layers: Tuple[DafotarLayer, ...]
    raw: dict

    @staticmethod
    def from_dict(raw: dict) -> "DafotarConfig":
        p = Problems("Dafotar config.json")
        V = need(raw, "vocab", int, p, required=True)
        W = need(raw, "width", int, p, required=True)
        norm = need(raw, "norm", dict, p, required=True) or {}
        eps = need(norm, "eps", float, p, required=True)
        streams = need(raw, "streams", int, p, default=None, allow_none=True)
        canon = need(raw, "canon", dict, p, default=None, allow_none=True)
        taps = need(canon, "taps", int, p, required=True) if canon is not None else None
        layers_raw = need(raw, "layers", list, p, required=True) or []
        p.raise_if_any()
        p.require(V > 0 and W > 0, f"'vocab' and 'width' must be positive, got {V} and {W}")
        p.require(eps > 0, f"'norm.eps' must be positive, got {eps}")
        p.require(streams is None or 1 <= streams <= 8, f"'streams' must lie in 1..8, got {streams}")
        p.require(taps is None or taps >= 1, f"'canon.taps' must be at least 1, got {taps}")
        p.require(len(layers_raw) > 0, "'layers' is empty")
        layers = []
        for i, lr in enumerate(layers_raw):
            q = Problems(f"layer {i}")
            if not isinstance(lr, dict):
                p.add(f"layer {i} must be an object")
                continue
            typ = need(lr, "type", str, q, required=True)
            mx = need(lr, "mixer", dict, q, required=True) or {}
            mlp = need(lr, "mlp", dict, q, default=None, allow_none=True)
            ff = None
            if mlp is not None:
                kind = need(mlp, "kind", str, q, default="dense")
                q.require(kind == "dense", f"mlp.kind must be 'dense', got {kind!r}")
                ff = need(mlp, "ff", int, q, required=True)
                q.require(ff is None or ff > 0, f"mlp.ff must be positive, got {ff}")
            heads = need(mx, "heads", int, q, required=True)
            dim = need(mx, "dim", int, q, required=True)
            vdim = need(mx, "vdim", int, q, required=True)
            if q.items:
                p.add(f"layer {i}: " + "; ".join(q.items))
                continue
            q.require(heads > 0 and dim > 0 and vdim > 0, "heads, dim and vdim must be positive")
            if typ == "attention":
                kvh = need(mx, "kv_heads", int, q, default=heads)
                scale = need(mx, "scale", float, q, required=True)
                mask = need(mx, "mask", dict, q, default=None, allow_none=True)
                window = need(mask, "size", int, q, required=True) if mask is not None else None
                rot = need(mx, "rot", dict, q, default=None, allow_none=True)
                base = need(rot, "base", float, q, required=True) if rot is not None else None
                dims = need(rot, "dims", int, q, default=dim) if rot is not None else 0
                src = need(mx, "kv_from", int, q, default=None, allow_none=True)
                if not q.items:
                    q.require(kvh > 0 and heads % kvh == 0, f"heads ({heads}) must be a multiple of kv_heads ({kvh})")
                    q.require(window is None or window > 0, f"mask.size must be positive, got {window}")
                    q.require(rot is None or (base > 0 and dims % 2 == 0 and 0 < dims <= dim),
                              f"rot.base must be positive and rot.dims even and in (0, dim], got {base} and {dims}")
                    q.require(rot is None or vdim % 2 == 0, f"rotated values need an even vdim, got {vdim}")
                    if src is not None:
                        ok = 0 <= src < i and src < len(layers) and layers[src].type == "attention" and \
                            layers[src].kv_from is None
                        q.require(ok, f"kv_from must name an earlier attention layer with keys of its own, got {src}")
                        if ok:
                            o = layers[src]
                            q.require((o.kv_heads, o.dim, o.vdim, o.rot_base, o.rot_dims) == (kvh, dim, vdim, base, dims),
                                      f"layer {src}'s key/value heads and rotation differ from this layer's")
                layers.append(DafotarLayer("attention", heads, dim, vdim, ff, kv_heads=kvh or heads, scale=scale or 1.0,
                                           window=window, rot_base=base, rot_dims=dims or 0, kv_from=src))
            elif typ == "mlstm":
                cap = need(mx, "gate_cap", float, q, required=True)
                q.require(cap is None or cap > 0, f"gate_cap must be positive, got {cap}")
                q.require(vdim <= 256, f"vdim up to 256 in an mlstm layer, got {vdim}")
                layers.append(DafotarLayer("mlstm", heads, dim, vdim, ff, gate_cap=cap or 1.0))
            else:
                q.add(f"unknown type {typ!r} (attention, mlstm)")
                layers.append(DafotarLayer(str(typ), heads, dim, vdim, ff))
            if q.items:
                p.add(f"layer {i}: " + "; ".join(q.items))
        p.raise_if_any()
        return DafotarConfig(V, W, eps, streams, taps, tuple(layers), dict(raw))

    def to_dict(self) -> dict:
        return dict(self.raw)


def dafotar_plan(c: DafotarConfig) -> ModelPlan:
    S = c.streams
    layers, order, owner_call = [], [], {}
    for i, l in enumerate(c.layers):
        pre = f"l{i}."
        if l.type == "attention":
            names = {"q": pre + "mix.q", "o": pre + "mix.o"}
            if l.kv_from is None:
                names.update(k=pre + "mix.k", v=pre + "mix.v")
            rotary = (RotarySpec(head_dim=l.dim, rotary_dim=l.rot_dims, theta=l.rot_base) if l.rot_base is not None
                      else NoPositionSpec())
            mixer = AttentionSpec(
                hidden_size=c.width, num_heads=l.heads, num_kv_heads=l.kv_heads, head_dim=l.dim, scale=l.scale,
                softcap=None, window=l.window, position=rotary, names=names, value_dim=l.vdim,
                q_norm=pre + "mix.q.norm", k_norm=(pre + "mix.k.norm") if l.kv_from is None else None,
                norm_eps=c.eps, head_scale=pre + "mix.temp", value_rotation=l.rot_base)
        else:
            mixer = MatrixMemorySpec(
                hidden_size=c.width, num_heads=l.heads, key_dim=l.dim, value_dim=l.vdim, gate_cap=l.gate_cap, eps=c.eps,
                names={"q": pre + "mix.q", "k": pre + "mix.k", "v": pre + "mix.v", "gate": pre + "mix.g",
                       "o": pre + "mix.o", "norm": pre + "mix.norm", "i": pre + "mix.i", "i_bias": pre + "mix.i.b",
                       "f": pre + "mix.f", "f_bias": pre + "mix.f.b"})
        ffn = None
        norms = {"pre_mixer": LayerNormSpec(c.width, c.eps, pre + "norm1", pre + "norm1.b")}
        if l.ff is not None:
            ffn = GatedMLPSpec(hidden_size=c.width, intermediate_size=l.ff, activation="relu",
                               names={r: f"{pre}mlp.{r}" for r in ("gate", "up", "down")})
            norms["pre_ffn"] = LayerNormSpec(c.width, c.eps, pre + "norm2", pre + "norm2.b")
        hc = {}
        if S is not None:
            for q in (1, 2) if ffn is not None else (1,):
                hc.update({f"in{q}": f"{pre}hc{q}.in", f"out{q}": f"{pre}hc{q}.out", f"mix{q}": f"{pre}hc{q}.mix"})
        conv = ShortConvSpec(c.width, c.taps, pre + "canon1") if c.taps is not None else None
        layers.append(StreamsBlockSpec(streams=S, mixer=mixer, ffn=ffn, norms=norms, conv=conv, names=hc))
        order.append(LayerCall(i, cache_of=l.kv_from if l.type == "attention" else None))
    return ModelPlan(
        architecture=NAME, hidden_size=c.width, vocab_size=c.vocab, max_position=MAX_POSITION,
        embedding=EmbeddingSpec(c.vocab, c.width, 1.0, "embed", copies=S or 1),
        layers=tuple(layers), order=tuple(order),
        final_norm=LayerNormSpec(c.width, c.eps, "final.norm", "final.norm.b", streams=S or 1),
        head=HeadSpec(c.vocab, c.width, None, "embed"),
        optional_prefixes=())


DAFOTAR = register_architecture(Architecture(
    name=NAME, config_from_dict=DafotarConfig.from_dict, plan=dafotar_plan, model_types=("dafotar",)))
