"""Softmax attention through a latent: queries, keys and values are made from low-rank vectors, and only the
key/value latent c (``kv_rank`` values, RMS-normed) and one rotated key part shared by all heads (``rot_dim`` values) are
cached per token, as ONE row of a single-plane paged cache.

    c_q = norm(W_dq h),  q = W_uq c_q = per head [dim plain | rot_dim rotated]
    W_dkv h = [kv_rank -> c = norm(.) | rot_dim -> k_rot, rotated, not normed]
    k_h = W_uk,h c,  v_h = W_uv,h c,  s = scale (q_plain . k_h + q_rot . k_rot),  causal softmax,
    out = W_o (concat_h(sum_j p_j v_hj) * sigmoid(W_g h))            (the gate is optional)

The keys and values are never made: with q' = W_uk,h^T q_plain the score is q' . c + q_rot . k_rot and the head's
result is W_uv,h (sum_j p_j c_j), so every head walks the same cached rows and two small products per head stand
before and after the walk.  Rotation: pairs (2i, 2i+1) of the first ``rot_dims`` entries of a rotated part turn by
position * base^(-2i/rot_dims), computed in float32.
"""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import CacheNeed, Mixer, register_part
from .linear import linear


def pair_frequencies(dims: int, base: float) -> torch.Tensor:
    """f_i = base^(-2i/dims), i < dims / 2, in float32 arithmetic."""
    i = torch.arange(dims // 2, dtype=torch.float32)
    return torch.pow(torch.tensor(float(base), dtype=torch.float32), -2.0 * i / dims).contiguous()


@register_part("mixer", "latent_attention")
class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, name, runtime, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int,
                 q_rank: int, kv_rank: int, softmax_scale: float, rot_base: float, rot_dims=None, norm_eps: float = 1e-6,
                 gate: bool = True):
        super().__init__(name, runtime)
        rot_dims = rot_dim if rot_dims is None else int(rot_dims)
        if min(num_heads, head_dim, value_dim, q_rank, kv_rank) <= 0 or rot_dim < 0:
            raise ValueError("latent attention: sizes must be positive")
        if kv_rank > ops.LATENT_MAX_RANK:
            raise ValueError("latent attention: a latent of %d values is beyond the kernel's %d" % (kv_rank, ops.LATENT_MAX_RANK))
        if rot_dims % 2 or not 0 <= rot_dims <= rot_dim:
            raise ValueError("latent attention: %d rotated dimensions do not fit a rotated part of %d" % (rot_dims, rot_dim))
        self.hidden_size, self.H, self.dim, self.E, self.dv = int(hidden_size), int(num_heads), int(head_dim), int(rot_dim), int(value_dim)
        self.Rq, self.R = int(q_rank), int(kv_rank)
        self.scale, self.eps, self.gate = float(softmax_scale), float(norm_eps), bool(gate)
        self.rot_dims = rot_dims
        self.freq = pair_frequencies(max(rot_dims, 2), rot_base).to(runtime.device)

    def cache_need(self):
        return CacheNeed("kv", n_kv_heads=1, head_dim=self.R + self.E, planes=1)

    def weight_specs(self):
        n, d, H = self.name, self.hidden_size, self.H
        pack = n + "down.packed"
        specs = {
            n + "dq": WeightSpec((self.Rq, d), pack=(pack, 0)),
            n + "dkv": WeightSpec((self.R + self.E, d), pack=(pack, 1)),
            n + "dq.norm": WeightSpec((self.Rq,), "vector"), n + "dkv.norm": WeightSpec((self.R,), "vector"),
            n + "uq": WeightSpec((H * (self.dim + self.E), self.Rq)),
            n + "uk": WeightSpec((H * self.dim, self.R)), n + "uv": WeightSpec((H * self.dv, self.R)),
            n + "o": WeightSpec((d, H * self.dv)),
        }
        if self.gate:
            specs[n + "g"] = WeightSpec((H * self.dv, d), pack=(pack, 2))
        return specs

    def load_weights(self, tensors):
        n, H = self.name, self.H
        packed = tensors.get(n + "down.packed")
        if packed is None:
            packed = torch.cat([tensors[n + s] for s in ["dq", "dkv"] + (["g"] if self.gate else [])], dim=0).contiguous()
        self.w_down = packed
        self.qn_w, self.kvn_w = tensors[n + "dq.norm"], tensors[n + "dkv.norm"]
        self.w_uq, self.w_o = tensors[n + "uq"], tensors[n + "o"]
        # per head: W_uk^T [kv_rank, dim] takes a plain query into the latent's space; W_uv [value_dim, kv_rank] takes the walk's result out
        self.w_uk_t = tensors[n + "uk"].view(H, self.dim, self.R).transpose(1, 2).contiguous()
        self.w_uv = tensors[n + "uv"].view(H, self.dv, self.R).contiguous()

    def portion_tile_rows(self):
        return ops.attention_prefill_tile_rows()       # the step lists its single-token rows: they take the walk kernel

    def _key_splits(self, ctx, n_rows) -> int:
        """Ways to split the keys of single-token rows, so that few rows still fill the chip: a function of the step's
        shape (such rows, rounded key count) alone."""
        if not n_rows or not ctx.max_context:
            return 1
        on_cores = ops.attention_latent_on_matrix_cores(self.runtime.dtype, self.R, self.E)
        blocks = n_rows * ((self.H + 31) // 32 if on_cores else (self.H + 3) // 4)
        steps = (int(ctx.max_context) + 31) // 32 if on_cores else (int(ctx.max_context) + 63) // 64
        return max(1, min(32, steps // 2, (2 * ctx.cu_count + blocks - 1) // blocks))

    def _attend(self, qa, walked, ctx, cache):
        """Single-token rows walk the cached rows (keys split so that few rows fill the chip); a portion of several
        tokens takes two matrix products over all its (token, head) rows (bfloat16; float32 walks everything)."""
        rt, T, H, R, E = self.runtime, qa.shape[0], self.H, self.R, self.E
        by_products = rt.dtype == torch.bfloat16 and rt.attention_impl == "auto" and ctx.n_decode_rows < T and (ctx.n_decode_rows > 0 or ctx.n_prefill_tiles > 0)
        if by_products:
            rows, n_rows = (None if ctx.decode_rows_identity else ctx.decode_rows), ctx.n_decode_rows
        else:
            rows, n_rows = None, T
        if n_rows:
            n_split = self._key_splits(ctx, n_rows) if (by_products or T == ctx.R) else 1
            part_acc = part_ml = None
            if n_split > 1:
                part_acc = ctx.ws.buffer("latent_part_acc", (T * H * n_split * R,), torch.float32)
                part_ml = ctx.ws.buffer("latent_part_ml", (T * H * n_split * 2,), torch.float32)
            ops.attention_latent(qa, walked, cache.k, cache.block_tables, ctx.token_req, ctx.positions, H, R, E, ctx.page_size,
                                 self.scale, n_split, part_acc, part_ml, row_list=rows, n_rows=n_rows)
        if not by_products:
            return
        from .linear import _library
        D = R + E
        for r, n in enumerate(ctx.req_len):
            if n < 2:
                continue
            row0, pos0 = ctx.req_start[r], ctx.req_pos[r]
            L = pos0 + n
            L_pad = (L + 15) // 16 * 16
            gathered = ctx.ws.buffer("latent_gathered", (L_pad, D), rt.dtype)
            gathered_t = ctx.ws.buffer("latent_gathered_t", (R, L_pad), rt.dtype)
            ops.latent_gather(cache.k, cache.block_tables[r], L, L_pad, ctx.page_size, R, gathered, gathered_t)
            per = max(1, min(n, (32 << 20) // (H * L_pad)))          # tokens per pass: the scores of a pass stay under 128 MB
            for q0 in range(0, n, per):
                qn = min(per, n - q0)
                cols = min(L_pad, (pos0 + q0 + qn + 15) // 16 * 16)     # keys beyond the pass's last token are not computed
                scores = ctx.ws.buffer("latent_scores", (qn * H, cols), torch.float32)
                _library(qa[row0 + q0:row0 + q0 + qn].view(qn * H, D), gathered[:cols], scores)
                probs = ctx.ws.buffer("latent_probs", (qn * H, cols), rt.dtype)
                ops.latent_softmax(scores, probs, H, pos0 + q0, self.scale)
                _library(probs, gathered_t[:, :cols], walked[row0 + q0:row0 + q0 + qn].view(qn * H, R))

    def forward(self, h, ctx, cache):
        rt, T, H, R, E = self.runtime, h.shape[0], self.H, self.R, self.E
        rows = ctx.ws.buffer("latent_rows", (T, self.w_down.shape[0]), rt.dtype)
        linear(h, self.w_down, rows, rt.gemm_impl, ws=ctx.ws)
        cq = ctx.ws.buffer("latent_cq", (T, self.Rq), rt.dtype)
        ops.latent_prep(rows, self.Rq, R, E, self.qn_w, self.kvn_w, self.eps, self.freq, self.rot_dims, ctx.positions, cq,
                        cache.k, cache.slots if cache.writes else None)
        q = ctx.ws.buffer("latent_q", (T, H * (self.dim + E)), rt.dtype)
        linear(cq, self.w_uq, q, rt.gemm_impl, ws=ctx.ws)
        qa = ctx.ws.buffer("latent_qa", (T, H * (R + E)), rt.dtype)
        ops.blocked_product(q.view(T, H, self.dim + E)[:, :, :self.dim], self.w_uk_t, qa.view(T, H, R + E)[:, :, :R])
        ops.latent_q_rotate(q, self.dim, E, R, H, self.freq, self.rot_dims, ctx.positions, qa)
        walked = ctx.ws.buffer("latent_walk", (T, H * R), rt.dtype)
        self._attend(qa, walked, ctx, cache)
        heads_out = ctx.ws.buffer("latent_heads", (T, H * self.dv), rt.dtype)
        gate = rows[:, self.Rq + R + E:].view(T, H, self.dv) if self.gate else None
        ops.blocked_product(walked.view(T, H, R), self.w_uv, heads_out.view(T, H, self.dv), gate=gate)
        y = ctx.ws.buffer("mixer_out", (T, self.hidden_size), rt.dtype)
        linear(heads_out, self.w_o, y, rt.gemm_impl, ws=ctx.ws)
        return y
