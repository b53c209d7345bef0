"""The Mezinex decoder in the engine against the plain implementation of its equations (plain_mezinex.py): each
mechanism's kernel alone, then whole models in the four replay modes and both dtypes, with sizes, counts and constants
that differ from layer to layer and from model to model, and greedy generation through the entry point."""
import json
import math
import os
import random

import pytest
import torch

import helpers as H
import plain_mezinex as P

pytestmark = pytest.mark.gpu

# bfloat16: a position where a group's values nearly cancel before its norm (or a gate sits at its edge) magnifies the
# rounding of the step before it many times over; float32 shows the same positions at 1e-6.  So single positions may
# be off by a good part of the largest logit, while few are, and the mean over the positions stays small.
BF16_WORST, BF16_SOME, BF16_MEAN = 0.5, 5e-2, 1.5e-2
DTYPES = [("float32", torch.float32, 5e-4), ("bfloat16", torch.bfloat16, BF16_WORST)]


def _compare(got, ref, dtype, tol, what, steps=None, median_only=False):
    worst = H.compare(got, ref, tol, what, steps)
    if dtype == torch.bfloat16:
        errs = sorted(float((row.double() - ref[rid][pos]).abs().max()) / float(ref[rid].abs().max()) for (rid, pos), row in got.items())
        assert errs[len(errs) // 2] <= BF16_MEAN, "%s: median error %.3g" % (what, errs[len(errs) // 2])
        if median_only:       # (drawn sizes: one position that magnifies rounding eighty times, in float32 too, taints what follows it in a recurrent state)
            return worst
        assert sum(errs) / len(errs) <= BF16_MEAN, "%s: mean error %.3g" % (what, sum(errs) / len(errs))
        assert sum(e > BF16_SOME for e in errs) <= max(2, 0.05 * len(errs)), "%s: %d of %d positions off by more than %.3g" % (
            what, sum(e > BF16_SOME for e in errs), len(errs), BF16_SOME)
    return worst


def _latent(heads, dim, rot_dim, rot_dims, vdim, q_rank, kv_rank, scale, base, ff):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank,
                                                  "kv_rank": kv_rank, "scale": scale, "rot": {"base": base, "dims": rot_dims}},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def _rglru(width, blocks, conv, ff):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def _mamba(heads, vdim, state, groups, norm_groups, conv, ff):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups,
                                        "conv": conv}, "mlp": {"kind": "dense", "ff": ff} if ff else None}


# Z1: three streams, the first two layers run three times, a pair table, a logit scale that is no power of two, a
# rotated part of which only half turns, as many groups as heads, one norm group, a layer without a feed-forward,
# eight heads (two walks of four).
Z1 = {"architecture": "Mezinex", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "logit_scale": 0.7, "streams": 3,
      "embedding": {"bigram": {"buckets": 257, "mul_prev": 31, "mul_cur": 7}}, "loop": {"start": 0, "stop": 2, "times": 3},
      "layers": [_mamba(4, 16, 24, 4, 1, 4, 128), _latent(3, 24, 16, 8, 40, 48, 40, 0.2, 10000.0, None),
                 _rglru(64, 4, 2, 80), _latent(8, 16, 8, 8, 16, 32, 64, 0.15, 500000.0, 64)]}
# Z2: one plain residual stream (no hyper-connections), no pair table, no loop, sizes that are no multiple of 4 or 8,
# a convolution of one tap, one block of gates, one group, three norm groups.
Z2 = {"architecture": "Mezinex", "vocab": 97, "width": 70, "norm": {"eps": 1e-6},
      "layers": [_rglru(36, 1, 1, None), _mamba(3, 20, 10, 1, 3, 3, 50), _latent(2, 10, 6, 6, 12, 20, 22, 0.3, 100.0, 60)]}
# Z3: hyper-connections over ONE stream, recurrent layers only (nothing is paged), a loop of a single pass.
Z3 = {"architecture": "Mezinex", "vocab": 150, "width": 64, "norm": {"eps": 1e-5}, "logit_scale": 3.0, "streams": 1,
      "embedding": {"bigram": {"buckets": 64, "mul_prev": 1000003, "mul_cur": 999983}}, "loop": {"start": 1, "stop": 2, "times": 1},
      "layers": [_rglru(48, 3, 4, 64), _mamba(2, 64, 16, 2, 2, 2, None)]}
# Z4: a latent of the 16-byte path with rotated and plain parts of equal size, a looped attention layer (two caches of
# one layer), four streams.
Z4 = {"architecture": "Mezinex", "vocab": 300, "width": 128, "norm": {"eps": 1e-5}, "logit_scale": 1.0, "streams": 4,
      "loop": {"start": 0, "stop": 1, "times": 2},
      "layers": [_latent(6, 32, 32, 32, 24, 64, 128, 0.1, 1000000.0, 96), _rglru(64, 2, 3, None)]}
CONFIGS = {"Z1": Z1, "Z2": Z2, "Z3": Z3, "Z4": Z4}
LENGTHS = {"Z1": [1, 2, 130, 61, 210, 37], "Z2": [3, 75, 1, 140, 18, 66], "Z3": [5, 160, 129, 64, 2, 90], "Z4": [2, 90, 17, 1, 260, 40]}


def _write_model(folder, cfg, seed):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    W = P.random_weights(cfg, seed)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in W.items()}, os.path.join(folder, "model.safetensors"))
    return W


_models, _engines, _plain = {}, {}, {}


def _model(tmp_path_factory, name):
    if name not in _models:
        folder = os.path.join(str(tmp_path_factory.getbasetemp()), "mezinex_" + name)
        _models[name] = (folder, _write_model(folder, CONFIGS[name], seed=len(name) + ord(name[-1])))
    return _models[name]


def _engine(tmp_path_factory, name, dtype, max_tokens, page_size=16, max_requests=4):
    from infinicore_infer_amd.engine import Engine
    key = (name, dtype, max_tokens, page_size, max_requests)
    if key not in _engines:
        folder, _ = _model(tmp_path_factory, name)
        _engines[key] = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=page_size, max_requests=max_requests)
    return _engines[key]


def _requests(name, seed=0):
    return {"r%d" % i: H.random_tokens(CONFIGS[name]["vocab"], n, seed * 100 + i) for i, n in enumerate(LENGTHS[name])}


def _reference(tmp_path_factory, name, requests):
    key = (name, tuple(sorted((k, tuple(v)) for k, v in requests.items())))
    if key not in _plain:
        _, W = _model(tmp_path_factory, name)
        _plain[key] = {rid: P.forward(CONFIGS[name], W, toks, torch.float64) for rid, toks in requests.items()}
    return _plain[key]


MODES = {
    "whole": H.trace_whole,
    "tail": lambda r: H.trace_last_one_by_one(r, tail=100),     # long decoding; recorded steps replay
    "chunks": H.trace_chunks,
    "mixed": H.trace_mixed,
}


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_replay_modes(tmp_path_factory, name, dname, dtype, tol, mode):
    """Prefill against token-by-token decoding, portions down to two tokens, unequal requests in one batch with pages
    and state slots used again: every position's logits against the plain implementation."""
    requests = _requests(name)
    steps, max_tokens = MODES[mode](requests)
    engine = _engine(tmp_path_factory, name, dtype, max_tokens)
    ref = _reference(tmp_path_factory, name, requests)
    got = H.run_trace(engine, steps)
    assert len(got) == sum(len(t) for t in requests.values())
    worst = _compare(got, ref, dtype, tol, "%s %s %s" % (name, dname, mode))
    print("worst error %.3g at %s (allowed %.3g)" % (worst[0], worst[1], tol))
    engine.cache.check_invariants()
    assert not engine.cache.requests
    for g in range(len(engine.groups)):
        assert engine.cache.free_pages(g) == engine.num_pages


@pytest.mark.parametrize("name,page_size", [("Z1", 64), ("Z4", 32)])
def test_other_page_sizes(tmp_path_factory, name, page_size):
    requests = _requests(name, seed=2)
    steps, max_tokens = H.trace_mixed(requests, seed=5)
    ref = _reference(tmp_path_factory, name, requests)
    engine = _engine(tmp_path_factory, name, torch.float32, max_tokens + 4 * page_size, page_size=page_size)
    H.compare(H.run_trace(engine, steps), ref, H.FP32_TOL, "%s page %d" % (name, page_size))
    engine.cache.check_invariants()


def test_recorded_decode_steps_equal_eager_ones(tmp_path_factory):
    """Long decoding: the same request decoded through recorded steps and eagerly gives the same logits; states and the
    remembered token move on exactly once per step, also in the step that is recorded."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    folder, W = _model(tmp_path_factory, "Z1")
    toks = H.random_tokens(Z1["vocab"], 200, 9)
    rows = {}
    for graphs in (True, False):
        eng = Engine.from_dir(folder, dtype=torch.float32, max_tokens=512, page_size=16, max_requests=2, use_graphs=graphs)
        eng.step([StepEntry("a", toks[:30], [])])
        out = []
        for t in toks[30:]:
            out.append(eng.step([StepEntry("a", [t], [0])]).float().cpu().clone())
        rows[graphs] = torch.cat(out)
        if graphs:
            assert eng.graph_replays > 100
    assert torch.equal(rows[True], rows[False])
    ref = P.forward(Z1, W, toks, torch.float64)[30:]
    assert float((rows[True].double() - ref).abs().max()) <= 1e-4 * float(ref.abs().max())


@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
def test_forked_requests_go_on_independently(tmp_path_factory, dname, dtype, tol):
    """Pages, recurrent states, convolution inputs and the remembered token are copied; both go on with different tokens."""
    from infinicore_infer_amd.engine import Engine, StepEntry
    folder, W = _model(tmp_path_factory, "Z1")
    eng = Engine.from_dir(folder, dtype=dtype, max_tokens=1024, page_size=16, max_requests=4)
    base = H.random_tokens(Z1["vocab"], 97, 1)
    tails = {"a": H.random_tokens(Z1["vocab"], 20, 2), "b": H.random_tokens(Z1["vocab"], 20, 3)}
    eng.step([StepEntry("a", base[:60], [])])
    eng.step([StepEntry("a", base[60:], [])])
    eng.fork("a", "b")
    got = {}
    for i in range(20):
        rows = eng.step([StepEntry(r, [tails[r][i]], [0]) for r in ("a", "b")]).float().cpu()
        for j, r in enumerate(("a", "b")):
            got[(r, len(base) + i)] = rows[j].clone()
    ref = {r: P.forward(Z1, W, base + tails[r], torch.float64) for r in tails}
    _compare(got, ref, dtype, tol, "fork %s" % dname)
    eng.free("a")
    eng.free("b")
    eng.cache.check_invariants()


# ---- the mechanisms alone ------------------------------------------------------------------------------------------
def _dev(t, dtype=None):
    return t.to(device="cuda", dtype=dtype if dtype is not None else t.dtype).contiguous()


def _i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device="cuda")


def test_pair_table_rows_and_the_remembered_token():
    """A sequence fed in portions beside another one: the pair rows are those of the whole sequence; the first token takes
    the last row; the hash is taken in 64 bits (multipliers near 2^20 would overflow 32)."""
    from infinicore_infer_amd.kernels import ops
    buckets, mp, mc, d, V = 1021, 1000003, 999983, 40, 50000
    seqs = {0: H.random_tokens(V, 23, 1), 1: H.random_tokens(V, 9, 2)}
    g = torch.Generator().manual_seed(0)
    table, pair = torch.randn(V, d, generator=g), torch.randn(buckets + 1, d, generator=g)
    want = {r: P.embed(s, table.double(), pair.double(), buckets, mp, mc) for r, s in seqs.items()}
    prev = torch.zeros(4, dtype=torch.int32, device="cuda")
    slots = {0: 2, 1: 0}
    cuts = [[(0, 5), (1, 1)], [(1, 2), (0, 1)], [(0, 2)], [(0, 15), (1, 6)]]
    at = {0: 0, 1: 0}
    for step in cuts:
        toks, pos, req = [], [], []
        for b, (r, n) in enumerate(step):
            toks += seqs[r][at[r]:at[r] + n]
            pos += list(range(at[r], at[r] + n))
            req += [b] * n
        T = len(toks)
        out = torch.empty(2, T, d, dtype=torch.float32, device="cuda")
        rows = torch.empty(T, dtype=torch.int32, device="cuda")
        st = _i32([slots[r] for r, _ in step])
        ops.pair_rows(_i32(toks), _i32(pos), _i32(req), st, prev, rows, buckets, mp, mc)
        ops.embed_streams(_i32(toks), _dev(table), out, rows=rows, pair_table=_dev(pair), token_req=_i32(req), state_slots=st,
                          prev_state=prev)
        o = 0
        for r, n in step:
            for s in range(2):
                assert torch.allclose(out[s, o:o + n].cpu().double(), want[r][at[r]:at[r] + n], atol=1e-6)
            o += n
            at[r] += n
    assert prev.tolist()[2] == seqs[0][-1] and prev.tolist()[0] == seqs[1][-1]


@pytest.mark.parametrize("S", [1, 2, 3, 5, 8])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_streams_write_read_and_norm_in_one_kernel(S, dtype):
    from infinicore_infer_amd.kernels import ops
    T, d, eps = 7, 100, 1e-5
    g = torch.Generator().manual_seed(S)
    xs = torch.randn(S, T, d, generator=g, dtype=torch.float64)
    y = torch.randn(T, d, generator=g).to(dtype).double()
    mix, ow, iw = (torch.eye(S) + 0.3 * torch.randn(S, S, generator=g)).double(), torch.randn(S, generator=g).double(), torch.randn(S, generator=g).double()
    nw = (1 + 0.2 * torch.randn(d, generator=g)).double()
    new = P.hyper_write(xs, y, mix, ow)
    u = P.hyper_read(new, iw)
    want_h = P.rms(u, eps) * nw
    x = _dev(xs, torch.float32)
    h = torch.empty(T, d, dtype=dtype, device="cuda")
    f = lambda t: _dev(t, torch.float32)
    ops.hc_step(x, y=_dev(y, dtype), mix=f(mix), out_w=f(ow), in_w=f(iw), norm_w=f(nw), eps=eps, h=h)
    assert torch.allclose(x.cpu().double(), new, atol=1e-5)
    assert torch.allclose(h.cpu().double(), want_h, atol=2e-5 if dtype == torch.float32 else 3e-2)
    # the write alone, and the read alone as a plain float32 sum
    x2 = _dev(xs, torch.float32)
    ops.hc_step(x2, y=_dev(y, dtype), mix=f(mix), out_w=f(ow))
    assert torch.equal(x2, x)
    total = torch.empty(T, d, dtype=torch.float32, device="cuda")
    ops.hc_step(x2, in_w=torch.ones(S, dtype=torch.float32, device="cuda"), h=total)
    assert torch.allclose(total.cpu().double(), new.sum(0), atol=1e-5)


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_convolution_over_portions_with_its_state(taps, dtype):
    """Two sequences cut into portions of 1, 2 and more tokens (shorter and longer than the taps), in state slots that are
    used again: the result is the whole sequence's convolution."""
    from infinicore_infer_amd.kernels import ops
    C, stride, off = 37, 50, 11
    g = torch.Generator().manual_seed(taps)
    w, b, ib = torch.randn(C, taps, generator=g), torch.randn(C, generator=g), torch.randn(C, generator=g)
    seqs = {r: torch.randn(n, C, generator=g).to(dtype) for r, n in ((0, 31), (1, 12), (2, 6))}
    want = {r: P.silu(P.causal_conv(s.double() + ib.double(), w.double(), b.double())) for r, s in seqs.items()}
    state = torch.zeros(3, off + (taps - 1) * C + 5, dtype=torch.float32, device="cuda")
    steps = [[(0, 1, 2)], [(0, 2, 2), (1, 5, 0)], [(1, 1, 0), (0, 9, 2)], [(0, 1, 2), (1, 6, 0)], [(0, 18, 2)], "free1", [(2, 2, 0)], [(2, 4, 0)]]
    at = {0: 0, 1: 0, 2: 0}
    for step in steps:
        if step == "free1":
            state[0].zero_()
            continue
        T = sum(n for _, n, _ in step)
        xin = torch.zeros(T, stride, dtype=dtype, device="cuda")
        req, starts, o = [], [0], 0
        for i, (r, n, _) in enumerate(step):
            xin[o:o + n, 3:3 + C] = seqs[r][at[r]:at[r] + n].cuda()
            req += [i] * n
            o += n
            starts.append(o)
        out = torch.empty(T, C, dtype=torch.float32, device="cuda")
        copy = torch.empty(T, C, dtype=dtype, device="cuda")
        ops.causal_conv(xin[:, 3:3 + C], _dev(w), _dev(b), out, state, off, _i32(req), _i32(starts), _i32([s for _, _, s in step]),
                        len(step), in_bias=_dev(ib), out_copy=copy, act="silu")
        o = 0
        for r, n, _ in step:
            assert torch.allclose(out[o:o + n].cpu().double(), want[r][at[r]:at[r] + n], atol=1e-5), (taps, r, at[r])
            assert torch.allclose(copy[o:o + n].cpu().double(), want[r][at[r]:at[r] + n], atol=1e-5 if dtype == torch.float32 else 3e-2)
            o += n
            at[r] += n


@pytest.mark.parametrize("chunk_len", [0, 1, 4, 7])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_linear_recurrence_over_portions(dtype, chunk_len):
    """(chunk_len > 0: every portion cut into chunks that run side by side.)  Two sequences in portions of 1, 2 and more tokens: gates from their pre-activations and biases, the decay, the
    state carried in its slot, the other branch's gelu; against the recurrence written out token by token."""
    from infinicore_infer_amd.kernels import ops
    width, bw, off = 24, 8, 3
    g = torch.Generator().manual_seed(5)
    lam = 1.5 * torch.randn(width, generator=g) - 1
    decay = (-8.0 * P.softplus(lam.double())).float()
    gb, yb_bias = torch.randn(2 * width, generator=g), torch.randn(width, generator=g)
    seqs = {}
    for r, n in ((0, 40), (1, 9)):
        seqs[r] = (torch.randn(n, 2 * width, generator=g), torch.randn(n, width, generator=g), torch.randn(n, width, generator=g).to(dtype))
    want = {}
    for r, (gates, u, yb) in seqs.items():
        pre = (gates.double() + gb.double()).view(-1, width // bw, 2, bw)
        rg, ig = torch.sigmoid(pre[:, :, 0]).reshape(-1, width), torch.sigmoid(pre[:, :, 1]).reshape(-1, width)
        S, rows = torch.zeros(width, dtype=torch.float64), []
        for t in range(len(u)):
            a = torch.exp(decay.double() * rg[t])
            S = a * S + torch.sqrt(1 - a * a) * ig[t] * u[t].double()
            rows.append(S * P.gelu_tanh(yb[t].double() + yb_bias.double()))
        want[r] = torch.stack(rows)
    state = torch.zeros(4, off + width + 2, dtype=torch.float32, device="cuda")
    at = {0: 0, 1: 0}
    for step in [[(0, 1, 3)], [(1, 2, 1), (0, 7, 3)], [(0, 2, 3), (1, 1, 1)], [(0, 30, 3), (1, 6, 1)]]:
        T = sum(n for _, n, _ in step)
        cat = lambda k: torch.cat([seqs[r][k][at[r]:at[r] + n] for r, n, _ in step]).cuda()
        starts = [0]
        for _, n, _ in step:
            starts.append(starts[-1] + n)
        out = torch.empty(T, width, dtype=dtype, device="cuda")
        chunks = None
        if chunk_len:
            most = max((n + chunk_len - 1) // chunk_len for _, n, _ in step)
            chunks = (chunk_len, most, torch.full((len(step) * most * width,), float("nan"), device="cuda"),
                      torch.full((len(step) * most * width,), float("nan"), device="cuda"))
        ops.rglru_scan(cat(0), gb.cuda(), cat(1), cat(2), yb_bias.cuda(), decay.cuda(), bw, out, state, off, _i32(starts),
                       _i32([s for _, _, s in step]), len(step), chunks=chunks)
        o = 0
        for r, n, _ in step:
            assert torch.allclose(out[o:o + n].cpu().double(), want[r][at[r]:at[r] + n], atol=2e-5 if dtype == torch.float32 else 3e-2)
            o += n
            at[r] += n


@pytest.mark.parametrize("chunk_len", [0, 1, 5])
@pytest.mark.parametrize("heads,Pd,N,G", [(4, 16, 24, 4), (3, 20, 10, 1), (2, 64, 16, 2), (6, 48, 32, 2), (1, 200, 8, 1), (2, 64, 128, 1), (1, 8, 300, 1)])
def test_state_space_recurrence_over_portions(heads, Pd, N, G, chunk_len):
    """(chunk_len > 0: every portion cut into chunks that run side by side.)  Step sizes from softplus, the decay, the matrix state per head carried in its slot, groups shared by heads, the
    skip term; a sequence in portions against the recurrence written out token by token."""
    from infinicore_infer_amd.kernels import ops
    inner, ch, off, n = heads * Pd, heads * Pd + 2 * G * N, 0, 21
    g = torch.Generator().manual_seed(heads + N)
    xbc = torch.randn(n, ch, generator=g)
    dt_raw = torch.randn(n, heads + 3, generator=g)
    dt_bias, a_log, dsk = 0.5 * torch.randn(heads, generator=g), 0.5 * torch.randn(heads, generator=g), torch.randn(heads, generator=g)
    neg_a = (-torch.exp(a_log.double())).float()
    x, B, C = xbc[:, :inner].double().view(n, heads, Pd), xbc[:, inner:inner + G * N].double().view(n, G, N), xbc[:, inner + G * N:].double().view(n, G, N)
    dt = P.softplus(dt_raw[:, :heads].double() + dt_bias.double())
    S, want = torch.zeros(heads, N, Pd, dtype=torch.float64), torch.zeros(n, heads, Pd, dtype=torch.float64)
    for t in range(n):
        for h in range(heads):
            gi = h // (heads // G)
            S[h] = torch.exp(neg_a[h].double() * dt[t, h]) * S[h] + dt[t, h] * torch.outer(B[t, gi], x[t, h])
            want[t, h] = S[h].T @ C[t, gi] + dsk[h].double() * x[t, h]
    state = torch.zeros(3, inner * N + 4, dtype=torch.float32, device="cuda")
    at = 0
    for m in (1, 2, 5, 1, 12):
        y = torch.empty(m, inner, dtype=torch.float32, device="cuda")
        chunks = None
        if chunk_len:
            most = (m + chunk_len - 1) // chunk_len
            chunks = (chunk_len, most, torch.full((most * inner * N,), float("nan"), device="cuda"),
                      torch.full((most * heads,), float("nan"), device="cuda"))
        ops.ssm_scan(xbc[at:at + m].cuda(), dt_raw[at:at + m, :heads].cuda(), dt_bias.cuda(), neg_a.cuda(), dsk.cuda(), heads, Pd, N, G, y,
                     state, off, _i32([0, m]), _i32([2]), 1, chunks=chunks)
        assert torch.allclose(y.cpu().double().view(m, heads, Pd), want[at:at + m], atol=1e-4, rtol=1e-5), (at, m)
        at += m


def test_gate_and_norm_in_groups():
    from infinicore_infer_amd.kernels import ops
    T, n, groups, eps = 5, 60, 3, 1e-5
    g = torch.Generator().manual_seed(2)
    y, z, w = torch.randn(T, n, generator=g), torch.randn(T, n + 4, generator=g), 1 + 0.2 * torch.randn(n, generator=g)
    v = y.double() * P.silu(z[:, :n].double())
    want = P.rms(v.view(T, groups, n // groups), eps).reshape(T, n) * w.double()
    out = torch.empty(T, n, dtype=torch.float32, device="cuda")
    ops.gated_group_norm(y.cuda(), z.cuda()[:, :n], w.cuda(), groups, eps, out)
    assert torch.allclose(out.cpu().double(), want, atol=1e-5)


@pytest.mark.parametrize("M,B,N,K", [(1, 3, 40, 24), (9, 2, 130, 70), (70, 4, 64, 16), (200, 1, 33, 129), (5, 2, 70, 64), (2, 3, 33, 40), (1, 3, 40, 21), (8, 40, 128, 512), (40, 3, 128, 64), (100, 2, 70, 48), (64, 5, 96, 16), (33, 2, 33, 80)])
@pytest.mark.parametrize("dtype,out_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32)])
def test_product_with_a_matrix_per_block_of_columns(M, B, N, K, dtype, out_dtype):
    from infinicore_infer_amd.kernels import ops
    g = torch.Generator().manual_seed(M + N)
    a = _dev(torch.randn(M, B * K + 5, generator=g), dtype)
    w = _dev(torch.randn(B, N, K, generator=g) / math.sqrt(K), dtype)
    gate = _dev(torch.randn(M, B * N, generator=g), dtype)
    out = torch.zeros(M, B * N + 3, dtype=out_dtype, device="cuda")
    av = a[:, :B * K].view(M, B, K)                 # rows strided: five more columns follow
    want = torch.einsum("mbk,bnk->mbn", av.double().cpu(), w.double().cpu())
    ops.blocked_product(av, w, out[:, :B * N].view(M, B, N))
    tol = 1e-5 if out_dtype == torch.float32 else 2e-2
    assert torch.allclose(out[:, :B * N].view(M, B, N).cpu().double(), want, atol=tol * float(want.abs().max()))
    assert float(out[:, B * N:].abs().max()) == 0
    if dtype == out_dtype:
        ops.blocked_product(av, w, out[:, :B * N].view(M, B, N), gate=gate.view(M, B, N))
        want = want * torch.sigmoid(gate.view(M, B, N).double().cpu())
        assert torch.allclose(out[:, :B * N].view(M, B, N).cpu().double(), want, atol=tol * float(want.abs().max()))


def _paged(rows_by_req, page_size, D, dtype, seed):
    """Rows of several requests in shuffled pages of one plane; pages nobody owns hold NaN."""
    n_pages = sum((len(r) + page_size - 1) // page_size for r in rows_by_req) + 3
    order = list(range(n_pages))
    random.Random(seed).shuffle(order)
    plane = torch.full((n_pages, 1, page_size, D), float("nan"), dtype=dtype)
    tables, k = [], 0
    for rows in rows_by_req:
        table = []
        for lo in range(0, len(rows), page_size):
            pg = order[k]
            k += 1
            n = min(page_size, len(rows) - lo)
            plane[pg, 0, :n] = rows[lo:lo + n].to(dtype)
            table.append(pg)
        tables.append(table)
    width = max(len(t) for t in tables)
    bt = torch.tensor([t + [0] * (width - len(t)) for t in tables], dtype=torch.int32)
    return plane.cuda(), bt.cuda()


@pytest.mark.parametrize("R,E,Hn,page", [(64, 32, 6, 16), (40, 8, 3, 16), (22, 6, 2, 32), (128, 64, 40, 64), (512, 64, 4, 16)])
@pytest.mark.parametrize("dname,dtype,tol", DTYPES)
def test_walk_over_the_latent_rows(R, E, Hn, page, dname, dtype, tol):
    """Queries at positions around page borders and steps of 64 keys, single tokens with their keys split several ways,
    and for every query one far key that its score singles out (the query is aligned with it): a lost or doubled key,
    or a key one off, changes the result by its whole weight."""
    from infinicore_infer_amd.kernels import ops
    D, scale = R + E, 0.5 / math.sqrt(R + E)
    g = torch.Generator().manual_seed(R + Hn)
    lens = [700, 130]
    rows = [torch.randn(n, D, generator=g).to(dtype).float() for n in lens]
    plane, bt = _paged(rows, page, D, dtype, seed=R)
    cases = []          # (request, position, far key)
    for pos in [0, 1, 15, 16, 17, 63, 64, 65, 127, 128, 300, 511, 512, 640, 699]:
        cases.append((0, pos, max(0, pos - 1 - (pos * 7) // 8)))
    for pos in [0, 31, 64, 129]:
        cases.append((1, pos, pos // 3))
    T = len(cases)
    q = torch.randn(T, Hn, D, generator=g)
    for i, (r, pos, far) in enumerate(cases):
        q[i, i % Hn] = rows[r][far] * (6.0 / scale / float(rows[r][far].pow(2).sum()))       # score 6 above a field near 0
    q = q.to(dtype)
    want = torch.zeros(T, Hn, R, dtype=torch.float64)
    for i, (r, pos, far) in enumerate(cases):
        k = rows[r][:pos + 1].double()
        p = torch.softmax(q[i].double() @ k.T * scale, dim=-1)
        want[i] = p @ k[:, :R]
        assert p[i % Hn, far] > 0.2
    qa = q.reshape(T, Hn * D).cuda()
    req, posd = _i32([c[0] for c in cases]), _i32([c[1] for c in cases])
    from infinicore_infer_amd.kernels.lib import get_lib
    on_cores = bool(get_lib().ic_attn_latent_on_matrix_cores(1 if dtype == torch.bfloat16 else 0, R, E))
    assert on_cores == (dtype == torch.bfloat16 and (R, E) in ((64, 32), (128, 64), (512, 64)))
    for n_split, vector in [(1, False), (3, False), (16, False)] + ([(1, True), (5, True)] if on_cores else []):
        out = torch.zeros(T, Hn * R, dtype=dtype, device="cuda")
        acc = torch.empty(T * Hn * n_split * R, dtype=torch.float32, device="cuda")
        ml = torch.empty(T * Hn * n_split * 2, dtype=torch.float32, device="cuda")
        ops.attention_latent(qa, out, plane, bt, req, posd, Hn, R, E, page, scale, n_split, acc, ml, vector_units=vector)
        got = out.view(T, Hn, R).cpu().double()
        assert torch.isfinite(got).all()
        err = (got - want).abs().amax(dim=(1, 2)) / want.abs().max()
        assert float(err.max()) <= (2e-5 if dtype == torch.float32 else 2e-2), (n_split, vector, cases[int(err.argmax())], float(err.max()))
    # a list of rows: only those are computed
    rows = _i32([3, 0, T - 1])
    out = torch.zeros(T, Hn * R, dtype=dtype, device="cuda")
    ops.attention_latent(qa, out, plane, bt, req, posd, Hn, R, E, page, scale, row_list=rows, n_rows=3)
    got = out.view(T, Hn, R).cpu().double()
    for i in range(T):
        if i in (3, 0, T - 1):
            assert float((got[i] - want[i]).abs().max()) <= (2e-5 if dtype == torch.float32 else 2e-2) * float(want.abs().max())
        else:
            assert float(got[i].abs().max()) == 0


@pytest.mark.parametrize("R,E,page,L,first", [(64, 32, 16, 150, 0), (40, 8, 32, 70, 33), (128, 64, 64, 5000, 4990), (24, 8, 16, 17, 3)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gathered_rows_and_the_masked_softmax_of_prompt_portions(R, E, page, L, first, dtype):
    """The pieces of the walk by matrix products: a request's rows out of shuffled pages (and their first R columns
    transposed, zero beyond the last key), and the softmax whose row m sees the keys up to first + m // heads."""
    from infinicore_infer_amd.kernels import ops
    D, Hn = R + E, 3
    g = torch.Generator().manual_seed(L)
    rows = [torch.randn(7, D, generator=g), torch.randn(L, D, generator=g).to(dtype).float()]
    plane, bt = _paged(rows, page, D, dtype, seed=L)
    L_pad = (L + 15) // 16 * 16
    got = torch.full((L_pad, D), float("nan"), dtype=dtype, device="cuda")
    got_t = torch.full((R, L_pad), float("nan"), dtype=dtype, device="cuda")
    ops.latent_gather(plane, bt[1], L, L_pad, page, R, got, got_t)
    assert torch.equal(got[:L].float().cpu(), rows[1]) and float(got[L:].float().abs().sum()) == 0
    assert torch.equal(got_t.float().cpu(), got[:, :R].float().cpu().T)
    n = L - first                      # the portion's tokens: positions first .. L - 1
    scores = torch.randn(n * Hn, L_pad, generator=g) * 3
    probs = torch.full((n * Hn, L_pad), float("nan"), dtype=dtype, device="cuda")
    ops.latent_softmax(scores.cuda(), probs, Hn, first, 0.37)
    want = torch.zeros(n * Hn, L_pad, dtype=torch.float64)
    for m in range(n * Hn):
        k = first + m // Hn + 1
        want[m, :k] = torch.softmax(scores[m, :k].double() * 0.37, dim=-1)
    assert torch.allclose(probs.float().cpu().double(), want, atol=1e-6 if dtype == torch.float32 else 4e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_norms_rotation_and_cache_write(dtype):
    """The query latent's norm, the key latent's norm and the rotated key part at positions up to 60,000, written to the
    slots given; the queries' rotated parts, of which only the first rot_dims entries turn."""
    from infinicore_infer_amd.kernels import ops
    from infinicore_infer_amd.parts.latent_attention import pair_frequencies
    Rq, R, E, dims, Hn, dim, base, eps = 20, 24, 12, 8, 3, 10, 10000.0, 1e-5
    T, page = 9, 16
    g = torch.Generator().manual_seed(1)
    rows = torch.randn(T, Rq + R + E + 7, generator=g).to(dtype)
    qn, kn = 1 + 0.2 * torch.randn(Rq, generator=g), 1 + 0.2 * torch.randn(R, generator=g)
    pos = torch.tensor([0, 1, 2, 17, 100, 1023, 4097, 33333, 60000])
    slots = torch.tensor([5, 40, 3, 17, 16, 31, 0, 63, 22], dtype=torch.int32)
    freq = pair_frequencies(dims, base).cuda()
    cache = torch.zeros(4, 1, page, R + E, dtype=dtype, device="cuda")
    cq = torch.empty(T, Rq, dtype=dtype, device="cuda")
    ops.latent_prep(rows.cuda(), Rq, R, E, qn.cuda(), kn.cuda(), eps, freq, dims, pos.to(torch.int32).cuda(), cq, cache, slots.cuda())
    r64 = rows.double()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert torch.allclose(cq.cpu().double(), P.rms(r64[:, :Rq], eps) * qn.double(), atol=tol)
    flat = cache.view(-1, R + E).cpu().double()[slots.long()]
    assert torch.allclose(flat[:, :R], P.rms(r64[:, Rq:Rq + R], eps) * kn.double(), atol=tol)
    # angles are float32 products of position and frequency: at position 60,000 that is 4e-3 rad from the exact angle
    assert torch.allclose(flat[:, R:], P.rotate_pairs(r64[:, Rq + R:Rq + R + E], pos, base, dims), atol=max(tol, 2e-2))
    assert torch.allclose(flat[:5, R:], P.rotate_pairs(r64[:5, Rq + R:Rq + R + E], pos[:5], base, dims), atol=max(tol, 1e-4))
    q = torch.randn(T, Hn * (dim + E), generator=g).to(dtype)
    qa = torch.zeros(T, Hn * (R + E), dtype=dtype, device="cuda")
    ops.latent_q_rotate(q.cuda(), dim, E, R, Hn, freq, dims, pos.to(torch.int32).cuda(), qa)
    want = P.rotate_pairs(q.double().view(T, Hn, dim + E)[:, :, dim:], pos, base, dims)
    got = qa.view(T, Hn, R + E).cpu().double()
    assert torch.allclose(got[:5, :, R:], want[:5], atol=max(tol, 1e-4)) and float(got[:, :, :R].abs().max()) == 0


# ---- generation through the entry point -------------------------------------------------------------------------------
def _plain_greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(P.forward(cfg, W, toks, torch.float64)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("name", ["Z1", "Z2", "Z3"])
def test_greedy_generation_through_the_entry_point_and_scheduler(tmp_path_factory, name):
    """Several prompts of unequal length through CausalLM.generate_batch (the scheduler: chunked prompts, continuous
    batching, recorded decode steps, decoding a step ahead of the host) in float32: the plain implementation's tokens."""
    from infinicore_infer_amd.causal_lm import CausalLM
    folder, W = _model(tmp_path_factory, name)
    cfg = CONFIGS[name]
    prompts = [H.random_tokens(cfg["vocab"], n, 40 + i) for i, n in enumerate([50, 3, 21])]
    model = CausalLM(folder, max_tokens=256, dtype=torch.float32, cache_tokens=1024, page_size=16, max_requests=4)
    outs = model.generate_batch(prompts, 10, max_batch_tokens=24, chunk_size=16)
    for p, o in zip(prompts, outs):
        assert o == _plain_greedy(cfg, W, p, 10)
    model.engine.cache.check_invariants()


def test_command_line_runs_the_design(tmp_path_factory):
    import subprocess
    import sys
    folder, W = _model(tmp_path_factory, "Z2")
    prompt = H.random_tokens(Z2["vocab"], 9, 77)
    r = subprocess.run([sys.executable, "-m", "infinicore_infer_amd.mezinex", "--amd", folder, "--dtype", "float32",
                        "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--max-tokens", "128"],
                       cwd=H.__file__.rsplit("/tests/", 1)[0], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    want = _plain_greedy(Z2, W, prompt, 6)
    assert " ".join(map(str, want)) in " ".join(r.stdout.split()), r.stdout[-2000:]


def test_command_line_with_random_weights(tmp_path):
    import subprocess
    import sys
    path = str(tmp_path / "config.json")
    with open(path, "w") as f:
        json.dump(Z4, f)
    r = subprocess.run([sys.executable, "-m", "infinicore_infer_amd.causal_lm", "--amd", "--random-weights", "--config", path,
                        "--prompt-len", "40", "--num-prompts", "3", "--max-new-tokens", "5", "--max-tokens", "256",
                        "--max-batch-tokens", "64", "--chunk-size", "32", "--weights-norm-std", "0.05"],
                       cwd=H.__file__.rsplit("/tests/", 1)[0], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert r.stdout.count("tokens[") == 3, r.stdout[-2000:]


# ---- configurations drawn from seeds -------------------------------------------------------------------------------------
def _drawn_config(seed):
    rng = random.Random(seed)
    width = rng.choice([34, 48, 64, 100])
    layers = []
    for _ in range(rng.choice([2, 3, 4])):
        kind = rng.choice(["latent_attention", "rglru", "mamba2"])
        ff = rng.choice([None, 24, 50, 128])
        if kind == "rglru":
            blocks = rng.choice([1, 2, 3, 5])
            layers.append(_rglru(blocks * rng.choice([4, 7, 16]), blocks, rng.choice([1, 2, 3, 4, 5]), ff))
        elif kind == "mamba2":
            groups = rng.choice([1, 2, 3])
            heads = groups * rng.choice([1, 2])
            vdim = rng.choice([8, 12, 32])
            ng = rng.choice([g for g in (1, 2, 3, 4, 6) if (heads * vdim) % g == 0 and heads * vdim // g >= 8])     # (a norm over a handful of values is a sign function: it magnifies any rounding)
            layers.append(_mamba(heads, vdim, rng.choice([4, 9, 16, 40]), groups, ng, rng.choice([1, 2, 3, 4]), ff))
        else:
            rot = rng.choice([2, 4, 8, 16])
            layers.append(_latent(rng.choice([1, 2, 4, 5, 7]), rng.choice([4, 8, 12, 32]), rot, rng.choice([d for d in (2, 4, 8, 16) if d <= rot]),
                                  rng.choice([4, 8, 20, 32]), rng.choice([8, 24, 40]), rng.choice([8, 12, 32, 56]),
                                  round(rng.uniform(0.05, 0.4), 3), rng.choice([100.0, 10000.0, 1e6]), ff))
    cfg = {"architecture": "Mezinex", "vocab": rng.choice([53, 128, 301]), "width": width, "norm": {"eps": rng.choice([1e-5, 1e-6, 1e-3])},
           "logit_scale": rng.choice([1.0, 0.5, 1.7]), "layers": layers}
    if rng.random() < 0.7:
        cfg["streams"] = rng.choice([1, 2, 3, 4])
    if rng.random() < 0.7:
        cfg["embedding"] = {"bigram": {"buckets": rng.choice([7, 100, 4099]), "mul_prev": rng.choice([1, 127, 65537]), "mul_cur": rng.choice([1, 17, 40503])}}
    if rng.random() < 0.6:
        a = rng.randrange(len(layers))
        cfg["loop"] = {"start": a, "stop": rng.randrange(a, len(layers) + 1), "times": rng.choice([1, 2, 3])}
    return cfg


@pytest.mark.parametrize("seed", list(range(10)))
def test_drawn_configurations(tmp_path_factory, seed):
    from infinicore_infer_amd.engine import Engine
    cfg = _drawn_config(seed)
    folder = os.path.join(str(tmp_path_factory.getbasetemp()), "mezinex_drawn_%d" % seed)
    W = _write_model(folder, cfg, seed)
    rng = random.Random(seed + 100)
    requests = {"r%d" % i: H.random_tokens(cfg["vocab"], n, seed * 10 + i)
                for i, n in enumerate([rng.choice([1, 2, 5, 40, 66, 129, 150]) for _ in range(5)])}
    ref = {rid: P.forward(cfg, W, toks, torch.float64) for rid, toks in requests.items()}
    steps, max_tokens = H.trace_mixed(requests, seed=seed)
    for dname, dtype, tol in DTYPES:
        engine = Engine.from_dir(folder, dtype=dtype, max_tokens=max_tokens, page_size=16, max_requests=4)
        # (tiny groups before a norm: one position of a bfloat16 run may flip; the mean and the count of such positions bound it)
        _compare(H.run_trace(engine, steps), ref, dtype, tol if dtype == torch.float32 else 1.5, "drawn %d %s" % (seed, dname), steps, median_only=True)
        engine.cache.check_invariants()
        assert not engine.cache.requests
