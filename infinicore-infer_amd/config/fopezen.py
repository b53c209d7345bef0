"""Typed configuration of the Fopezen decoder, read from config.json.

Keys: ``architecture`` ("Fopezen"), ``vocab``, ``width``, ``norm.eps`` and ``layers``: a list whose entries give
``type`` ("attention" or "attention_2"), ``mixer`` (heads, kv_heads, dim, vdim, scale, mask {size, keep_first},
v_mix) and ``mlp`` ({kind: "dense", ff} or null).  Tensor names: ``embed``, ``final.norm``, and per layer i
``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.up`` / ``.down``.

The design, layer by layer (x the float32 residual stream, r(z) = z / sqrt(mean(z^2) + eps)):
  x_0 = E[token] + s(p),  s(p)[2i] = sin(p 10000^(-2i/width)),  s(p)[2i+1] = cos(p 10000^(-2i/width))
  x <- x + r(mixer(x)) (1 + w_norm1);   x <- x + r(W_down relu(W_up x)^2) (1 + w_norm2)   (second half if mlp)
  logits = E (r(x) (1 + w_final))
Both mixers are attention without rotation over a window of ``mask.size`` keys plus the first ``mask.keep_first``
keys, with biases on q, k, v, grouped key/value heads, a query/key norm with a plain weight and value mixing with
the first mixing layer's values.  "attention": the norm per head, a sink in the softmax's denominator, an output
gate sigmoid(W_g x) and a bias on the output projection.  "attention_2": the norm over the whole projection, a
plain softmax, no gate, no output bias.
"""
from dataclasses import dataclass, field
from typing import List, Optional

from .registry import ConfigError, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, default_schedule

SINUSOID_BASE = 10000.0
DEFAULT_CONTEXT = 65536        # the design has no limit of its own; a serving cap (max_tokens) replaces this

_MIXER_KINDS = {
    # type -> (qk_norm, sink, gate, out_bias)
    "attention": ("head", True, True, True),
    "attention_2": ("row", False, False, False),
}


@dataclass
class FopezenMixer:
    kind: str
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]
    keep_first: int
    v_mix: bool


@dataclass
class FopezenLayer:
    mixer: FopezenMixer
    ff: Optional[int]            # None: the layer has no feed-forward


def _need(d: dict, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError("config.json lacks %s%s" % (where, key))
    return d[key]


@dataclass
class FopezenConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: List[FopezenLayer]
    context_cap: Optional[int] = None
    eos_token_id: List[int] = field(default_factory=list)
    bos_token_id: Optional[int] = None
    model_type: str = "Fopezen"

    @classmethod
    def from_dict(cls, cfg: dict, max_tokens: Optional[int] = None) -> "FopezenConfig":
        layers = []
        raw_layers = _need(cfg, "layers", "")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        for i, l in enumerate(raw_layers):
            where = "layers[%d]." % i
            kind = _need(l, "type", where)
            if kind not in _MIXER_KINDS:
                raise ConfigError("%stype %r: this design has the mixers %s" % (where, kind, ", ".join(sorted(_MIXER_KINDS))))
            m = _need(l, "mixer", where)
            mw = where + "mixer."
            mask = m.get("mask") or {}
            size = mask.get("size")
            mixer = FopezenMixer(
                kind=kind, heads=int(_need(m, "heads", mw)), kv_heads=int(m.get("kv_heads") or m["heads"]),
                dim=int(_need(m, "dim", mw)), vdim=int(m.get("vdim") or m["dim"]), scale=float(_need(m, "scale", mw)),
                window=int(size) if size else None, keep_first=int(mask.get("keep_first") or 0),
                v_mix=bool(m.get("v_mix", False)))
            mlp = l.get("mlp")
            ff = None
            if mlp:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError("%smlp.kind %r: this design's feed-forward is dense" % (where, mlp.get("kind")))
                ff = int(_need(mlp, "ff", where + "mlp."))
            layers.append(FopezenLayer(mixer, ff))
        eos = cfg.get("eos_token_id", [])
        eos = [] if eos is None else ([eos] if isinstance(eos, int) else list(eos))
        out = cls(vocab_size=int(_need(cfg, "vocab", "")), hidden_size=int(_need(cfg, "width", "")),
                  norm_eps=float(_need(_need(cfg, "norm", ""), "eps", "norm.")), layers=layers,
                  context_cap=int(max_tokens) if max_tokens is not None else None,
                  eos_token_id=[int(e) for e in eos], bos_token_id=cfg.get("bos_token_id"))
        out.validate()
        return out

    def validate(self) -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if self.context_cap is not None and self.context_cap <= 0:
            raise ConfigError("max_tokens (the cap on the context) must be positive")
        mixing = [l.mixer for l in self.layers if l.mixer.v_mix]
        if len({(m.kv_heads, m.vdim) for m in mixing}) > 1:
            raise ConfigError("layers that mix values must agree in kv_heads and vdim")
        for i, l in enumerate(self.layers):
            m = l.mixer
            if min(m.heads, m.kv_heads, m.dim, m.vdim) <= 0 or m.heads % m.kv_heads:
                raise ConfigError("layers[%d]: heads (%d) must be a positive multiple of kv_heads (%d); dim and vdim positive"
                                  % (i, m.heads, m.kv_heads))
            if m.window is not None and m.window <= 0 or m.keep_first < 0:
                raise ConfigError("layers[%d]: mask.size must be positive and mask.keep_first not negative" % i)
            if l.ff is not None and l.ff <= 0:
                raise ConfigError("layers[%d]: mlp.ff must be positive" % i)

    @property
    def max_positions(self) -> int:
        return self.context_cap if self.context_cap is not None else DEFAULT_CONTEXT

    context_is_open = True      # positions are bounded by the serving cap or the cache pool only

    @property
    def default_dtype(self) -> str:
        return "bfloat16"

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    def to_dict(self) -> dict:
        layers = []
        for l in self.layers:
            m = l.mixer
            layers.append({
                "type": m.kind,
                "mixer": {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
                          "mask": {"size": m.window, "keep_first": m.keep_first} if m.window else None, "v_mix": m.v_mix},
                "mlp": {"kind": "dense", "ff": l.ff} if l.ff is not None else None})
        return {"architecture": "Fopezen", "vocab": self.vocab_size, "width": self.hidden_size,
                "norm": {"eps": self.norm_eps}, "layers": layers}

    def model_spec(self) -> ModelSpec:
        d, eps = self.hidden_size, self.norm_eps
        norm = lambda tensor: PartSpec("rmsnorm", "", {"size": d, "eps": eps, "weight_offset": 1.0, "tensor": tensor})
        layers = []
        first_mix = next((i for i, l in enumerate(self.layers) if l.mixer.v_mix), None)
        for i, l in enumerate(self.layers):
            p, m = "l%d." % i, l.mixer
            qk_norm, sink, gate, out_bias = _MIXER_KINDS[m.kind]
            layers.append(LayerSpec(
                block=PartSpec("outnorm_residual", p, {}),
                mixer=PartSpec("span_attention", p + "mix.", {
                    "hidden_size": d, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
                    "value_dim": m.vdim, "softmax_scale": m.scale, "window": m.window, "keep_first": m.keep_first,
                    "sink": sink, "qk_norm": qk_norm, "qk_norm_eps": eps, "qkv_bias": True, "out_bias": out_bias,
                    "gate": gate, "value_mix": (None if not m.v_mix else "keep" if i == first_mix else "mix"),
                    "value_mix_optional": True}),
                mixer_norm=norm(p + "norm1"),
                feed_forward=None if l.ff is None else PartSpec("dense_act", p + "mlp.", {
                    "hidden_size": d, "intermediate_size": l.ff, "activation": "relu2"}),
                feed_forward_norm=None if l.ff is None else norm(p + "norm2")))
        return ModelSpec(
            architecture=self.model_type, vocab_size=self.vocab_size, hidden_size=d, max_positions=self.max_positions,
            embedding=PartSpec("embedding", "embed.", {"vocab_size": self.vocab_size, "hidden_size": d, "tensor": "embed",
                                                       "sinusoid_base": SINUSOID_BASE}),
            layers=layers, schedule=default_schedule(len(layers)),
            final_norm=norm("final.norm"),
            head=PartSpec("lm_head", "head.", {"vocab_size": self.vocab_size, "hidden_size": d, "tensor": "embed"}),
            eos_token_ids=list(self.eos_token_id), bos_token_id=self.bos_token_id)


register_architecture(["Fopezen", "fopezen"], FopezenConfig)
