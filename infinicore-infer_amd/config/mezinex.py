"""Typed configuration of the Mezinex decoder, read from config.json.

Keys: ``architecture`` ("Mezinex"), ``vocab``, ``width``, ``norm.eps``, ``logit_scale``, ``streams`` (residual
streams joined by hyper-connections; absent: one stream with plain residual sums), ``embedding.bigram`` {buckets,
mul_prev, mul_cur} (a hashed table of token pairs added to the embedding; absent: none), ``loop`` {start, stop, times}
(layers start..stop-1 run ``times`` times in a row with the same weights, every pass with a cache or state of its own)
and ``layers``: a list whose entries give ``type`` ("latent_attention", "rglru" or "mamba2"), ``mixer`` (the sizes of
that mixer) and ``mlp`` ({kind: "dense", ff} or null).  Tensor names: ``embed``, ``bigram``, ``final.norm``, ``head`` and
per layer i ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.gate`` / ``.up`` / ``.down``, ``l<i>.hc<q>.in`` /
``.out`` / ``.mix``.

The design, layer by layer (x_1..x_S the float32 residual streams, r(z) = z / sqrt(mean(z^2) + eps)):
  x_s = E[token] + P[(prev * mul_prev + token * mul_cur) mod buckets]   (P's last row for a sequence's first token)
  sublayer q of a layer: u = sum_s in_q[s] x_s;  y = f_q(r(u) w_q);  x_t <- sum_s mix_q[s, t] x_s + out_q[t] y
  f_1 is the layer's mixer, f_2 (if the layer has one) W_down (silu(W_gate h) * (W_up h))
  logits = logit_scale * W_head (r(sum_s x_s) w_final)
The mixers are described where they are built: ``parts/latent_attention.py`` and ``parts/recurrent.py``.
"""
from dataclasses import dataclass, field
from typing import List, Optional

from .registry import ConfigError, register_architecture
from .spec import ExecEntry, LayerSpec, ModelSpec, PartSpec

DEFAULT_CONTEXT = 65536        # the design has no limit of its own; a serving cap (max_tokens) replaces this
RGLRU_DECAY_SCALE = 8.0        # log a = -8 r softplus(lam): fixed by the design
MIXERS = ("latent_attention", "rglru", "mamba2")


def _need(d, key: str, where: str):
    if not isinstance(d, dict) or key not in d:
        raise ConfigError("config.json lacks %s%s" % (where, key))
    return d[key]


@dataclass
class MezinexLayer:
    kind: str
    mixer: dict                  # the mixer's sizes as config.json gives them
    ff: Optional[int]            # None: the layer has no feed-forward


@dataclass
class MezinexConfig:
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: List[MezinexLayer]
    logit_scale: float = 1.0
    streams: Optional[int] = None                 # None: plain residual sums
    bigram: Optional[dict] = None                 # {buckets, mul_prev, mul_cur}
    loop: Optional[dict] = None                   # {start, stop, times}
    context_cap: Optional[int] = None
    eos_token_id: List[int] = field(default_factory=list)
    bos_token_id: Optional[int] = None
    model_type: str = "Mezinex"

    @classmethod
    def from_dict(cls, cfg: dict, max_tokens: Optional[int] = None) -> "MezinexConfig":
        raw_layers = _need(cfg, "layers", "")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, l in enumerate(raw_layers):
            where = "layers[%d]." % i
            kind = _need(l, "type", where)
            if kind not in MIXERS:
                raise ConfigError("%stype %r: this design has the mixers %s" % (where, kind, ", ".join(MIXERS)))
            m = _need(l, "mixer", where)
            if not isinstance(m, dict):
                raise ConfigError("%smixer must be an object" % where)
            mlp = l.get("mlp")
            ff = None
            if mlp:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError("%smlp.kind %r: this design's feed-forward is dense" % (where, mlp.get("kind")))
                ff = int(_need(mlp, "ff", where + "mlp."))
            layers.append(MezinexLayer(kind, dict(m), ff))
        big = (cfg.get("embedding") or {}).get("bigram")
        if big:
            big = {k: int(_need(big, k, "embedding.bigram.")) for k in ("buckets", "mul_prev", "mul_cur")}
        loop = cfg.get("loop")
        if loop:
            loop = {k: int(_need(loop, k, "loop.")) for k in ("start", "stop", "times")}
        eos = cfg.get("eos_token_id", [])
        eos = [] if eos is None else ([eos] if isinstance(eos, int) else list(eos))
        out = cls(vocab_size=int(_need(cfg, "vocab", "")), hidden_size=int(_need(cfg, "width", "")),
                  norm_eps=float(_need(_need(cfg, "norm", ""), "eps", "norm.")), layers=layers,
                  logit_scale=float(cfg.get("logit_scale", 1.0)),
                  streams=int(cfg["streams"]) if cfg.get("streams") is not None else None,
                  bigram=big or None, loop=loop or None,
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
        if self.streams is not None and not 1 <= self.streams <= 8:
            raise ConfigError("streams must lie in 1..8")
        if self.bigram and (self.bigram["buckets"] <= 0 or min(self.bigram["mul_prev"], self.bigram["mul_cur"]) < 0):
            raise ConfigError("embedding.bigram: buckets must be positive, the multipliers not negative")
        n = len(self.layers)
        if self.loop and not (0 <= self.loop["start"] <= self.loop["stop"] <= n and self.loop["times"] >= 1):
            raise ConfigError("loop: 0 <= start <= stop <= %d layers and times >= 1 (got %r)" % (n, self.loop))
        for i, l in enumerate(self.layers):
            if l.ff is not None and l.ff <= 0:
                raise ConfigError("layers[%d]: mlp.ff must be positive" % i)
            self._mixer_params(i, l)          # names what is missing

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

    def run_order(self) -> List[int]:
        """Layer indices in the order they run: the looped stretch ``times`` times in a row."""
        n = len(self.layers)
        if not self.loop:
            return list(range(n))
        a, b, times = self.loop["start"], self.loop["stop"], self.loop["times"]
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))

    def to_dict(self) -> dict:
        out = {"architecture": "Mezinex", "vocab": self.vocab_size, "width": self.hidden_size,
               "norm": {"eps": self.norm_eps}, "logit_scale": self.logit_scale,
               "layers": [{"type": l.kind, "mixer": dict(l.mixer),
                           "mlp": {"kind": "dense", "ff": l.ff} if l.ff is not None else None} for l in self.layers]}
        if self.streams is not None:
            out["streams"] = self.streams
        if self.bigram:
            out["embedding"] = {"bigram": dict(self.bigram)}
        if self.loop:
            out["loop"] = dict(self.loop)
        return out

    def _mixer_params(self, i: int, l: MezinexLayer) -> PartSpec:
        d, m, where = self.hidden_size, l.mixer, "layers[%d].mixer." % i
        name = "l%d.mix." % i
        get = lambda k: _need(m, k, where)
        if l.kind == "rglru":
            return PartSpec("rglru", name, {"hidden_size": d, "width": int(get("width")), "blocks": int(get("blocks")),
                                            "conv_taps": int(get("conv")), "decay_scale": RGLRU_DECAY_SCALE})
        if l.kind == "mamba2":
            return PartSpec("mamba2", name, {
                "hidden_size": d, "heads": int(get("heads")), "head_dim": int(get("vdim")), "state_dim": int(get("state")),
                "groups": int(get("groups")), "conv_taps": int(get("conv")), "norm_groups": int(get("norm_groups")),
                "norm_eps": self.norm_eps})
        rot = get("rot")
        return PartSpec("latent_attention", name, {
            "hidden_size": d, "num_heads": int(get("heads")), "head_dim": int(get("dim")), "rot_dim": int(get("rot_dim")),
            "value_dim": int(get("vdim")), "q_rank": int(get("q_rank")), "kv_rank": int(get("kv_rank")),
            "softmax_scale": float(get("scale")), "rot_base": float(_need(rot, "base", where + "rot.")),
            "rot_dims": int(_need(rot, "dims", where + "rot.")), "norm_eps": self.norm_eps, "gate": True})

    def model_spec(self) -> ModelSpec:
        d, eps = self.hidden_size, self.norm_eps
        norm = lambda tensor: PartSpec("rmsnorm", "", {"size": d, "eps": eps, "tensor": tensor})
        layers = []
        for i, l in enumerate(self.layers):
            p = "l%d." % i
            block = (PartSpec("hyper_connections", p, {"streams": self.streams}) if self.streams is not None
                     else PartSpec("prenorm_residual", p, {}))
            layers.append(LayerSpec(
                block=block, mixer=self._mixer_params(i, l), mixer_norm=norm(p + "norm1"),
                feed_forward=None if l.ff is None else PartSpec("swiglu", p + "mlp.", {
                    "hidden_size": d, "intermediate_size": l.ff, "gate_name": "gate", "up_name": "up", "down_name": "down"}),
                feed_forward_norm=None if l.ff is None else norm(p + "norm2")))
        big = self.bigram or {}
        schedule = [ExecEntry(layer=li, cache=run, writes_cache=True) for run, li in enumerate(self.run_order())]
        return ModelSpec(
            architecture=self.model_type, vocab_size=self.vocab_size, hidden_size=d, max_positions=self.max_positions,
            embedding=PartSpec("pair_embedding", "embed.", {
                "vocab_size": self.vocab_size, "hidden_size": d, "tensor": "embed", "pair_tensor": "bigram" if big else None,
                "buckets": big.get("buckets", 0), "mul_prev": big.get("mul_prev", 0), "mul_cur": big.get("mul_cur", 0),
                "streams": self.streams or 1}),
            layers=layers, schedule=schedule, final_norm=norm("final.norm"),
            head=PartSpec("lm_head", "head.", {"vocab_size": self.vocab_size, "hidden_size": d, "tensor": "head",
                                               "logit_scale": self.logit_scale}),
            eos_token_ids=list(self.eos_token_id), bos_token_id=self.bos_token_id,
            residual_streams=self.streams or 1)


register_architecture(["Mezinex", "mezinex"], MezinexConfig)
