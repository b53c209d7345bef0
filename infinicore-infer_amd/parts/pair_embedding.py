"""Token embedding with a hashed table of token pairs, written into one or several residual streams.

x[t] = E[token_t] + P[(token_(t-1) * mul_prev + token_t * mul_cur) mod buckets]; a sequence's first token takes the
table's last row (row ``buckets``).  The token before a step's first one is part of the sequence's state: an int32
per request that the engine keeps with the mixers' states (zero for a new request, copied by a fork).  Without a
pair table it is the plain gather.  With ``streams`` > 1 every stream starts as a copy of the sum.
"""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import CacheNeed, Part, register_part


@register_part("embedding", "pair_embedding")
class PairEmbedding(Part):
    graph_safe = True
    category = "embedding"
    takes_context = True

    def __init__(self, name, runtime, vocab_size: int, hidden_size: int, tensor=None, pair_tensor=None, buckets: int = 0,
                 mul_prev: int = 0, mul_cur: int = 0, streams: int = 1):
        super().__init__(name, runtime)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.tensor = tensor if tensor is not None else name + "weight"
        self.pair_tensor = pair_tensor
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)
        if pair_tensor is not None and (self.buckets <= 0 or self.mul_prev < 0 or self.mul_cur < 0):
            raise ValueError("pair embedding: buckets must be positive and the multipliers not negative")
        self.streams = int(streams)
        self.table = self.pair_table = None

    def cache_need(self):
        return CacheNeed("state", state_shape=(1,), state_dtype=torch.int32) if self.pair_tensor is not None else CacheNeed()

    def weight_specs(self):
        specs = {self.tensor: WeightSpec((self.vocab_size, self.hidden_size), "matrix")}
        if self.pair_tensor is not None:
            specs[self.pair_tensor] = WeightSpec((self.buckets + 1, self.hidden_size), "matrix")
        return specs

    def load_weights(self, tensors):
        self.table = tensors[self.tensor]
        if self.pair_tensor is not None:
            self.pair_table = tensors[self.pair_tensor]
            if self.pair_table.dtype != self.table.dtype:
                self.pair_table = self.pair_table.to(self.table.dtype)

    def forward(self, tokens, x, ctx):
        T = tokens.numel()
        out = x.view(self.streams, T, self.hidden_size)
        if self.pair_table is None:
            ops.embed_streams(tokens, self.table, out)
            return None
        prev = ctx.embedding_state
        if prev is None:
            raise RuntimeError("the pair embedding needs the engine's per-request state (the token before a step's first)")
        prev = prev.view(-1)
        rows = ctx.ws.buffer("pair_rows", (T,), torch.int32)
        ops.pair_rows(tokens, ctx.positions, ctx.token_req, ctx.state_slots, prev, rows, self.buckets, self.mul_prev, self.mul_cur)
        ops.embed_streams(tokens, self.table, out, rows=rows, pair_table=self.pair_table, token_req=ctx.token_req,
                          state_slots=ctx.state_slots, prev_state=prev)
        return None
