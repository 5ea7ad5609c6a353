"""Meronex on the GPU: every mechanism's kernel against the plain implementation's function, then whole models through
the trace replay (the engine's step function, cache manager and kernels) under every schedule, far keys, long decoding,
and greedy generation through the entry point with and without captured steps."""
import json
import os
import subprocess
import sys

import pytest
import torch

from tests import meronex_cases as mc
from tests import replay_cases as rc
from tests.gpu_util import close, require_gpu
from tests.plain import meronex_plain as plain
from tests.test_gpu_sodedra import DT, TOL, i32, rnd, two_steps

pytestmark = pytest.mark.gpu


def compare(got, ref, dtype, what):
    """float32: every logit within a small tolerance.  bfloat16: a row's error, root mean square over the vocabulary,
    against the row's own root mean square, in the median and for nine rows in ten.  The bounds are what rounding alone
    does to these models, measured with exact arithmetic between bfloat16 roundings at the operations' edges (0.03 to
    0.04 in the median and 0.1 to 0.2 at the ninth decile, more where one expert of few is chosen): every layer has two
    gated sublayers, every feed-forward a router whose close call picks another expert (with one choice, all of the
    sublayer's result changes), and every mixer a state that carries such a token's effect on to all later ones; float32
    holds every row, and every kernel is held in bfloat16 by itself above."""
    if dtype == "float32":
        return rc.compare(got, ref, what=what, **TOL["float32"])
    assert got, "the replay wrote no logits"
    rel = []
    for (rid, pos), row in sorted(got.items(), key=lambda kv: (str(kv[0][0]), kv[0][1])):
        want = ref[rid][pos].double()
        err = torch.from_numpy(row).double() - want
        assert bool(torch.isfinite(err).all()), "%s: request %r position %d is not finite" % (what, rid, pos)
        rel.append(float(err.pow(2).mean().sqrt() / want.pow(2).mean().sqrt()))
    rel = torch.tensor(rel)
    assert float(rel.median()) < 0.08 and float(rel.quantile(0.9)) < 0.5, \
        "%s: rows are off by %.3f of their size in the median, %.3f at the ninth decile" % (what, float(rel.median()), float(rel.quantile(0.9)))


# ---- mechanisms --------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,H,groups", [(13, 50, 5), (5, 2048, 4), (70, 1100, 1), (9, 42, 7), (3, 8192, 2)])
def test_norm_in_groups_and_result_gate(dtype, T, H, groups):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(2)
    resid, a, w = rnd(g, T, H), rnd(g, T, H).to(DT[dtype]), (1.0 + rnd(g, H, std=0.3)).to(DT[dtype])
    # one group far larger than the others: a norm over the whole row would flatten it
    resid[:, :H // groups] *= 30.0
    r = resid.float().to(dev)
    out = ops.add_rms_norm(r, a.to(dev), w.to(dev), 1e-5, DT[dtype], groups=groups)
    x = resid.float().double() + a.double()
    close(r, x, torch.float32, what="stream after the addend")
    close(out, plain.grouped_norm(x, w.double(), 1e-5, groups), DT[dtype], what="norm in %d groups" % groups)
    rows = i32([T - 1, 0], dev)
    r2 = resid.float().to(dev)
    out2 = ops.add_rms_norm(r2, a.to(dev), w.to(dev), 1e-5, DT[dtype], rows, groups=groups)
    close(out2, plain.grouped_norm(x, w.double(), 1e-5, groups)[[T - 1, 0]], DT[dtype], what="norm of chosen rows")
    assert torch.equal(r2.cpu(), resid.float())
    y, pre, b = rnd(g, T, H).to(DT[dtype]), rnd(g, T, H + 7).to(DT[dtype]), rnd(g, H).to(DT[dtype])
    got = ops.sigmoid_gate(y.to(dev), pre.to(dev)[:, 3:3 + H], b.to(dev), 0.45)
    gated = y.double() * 0.45 * torch.sigmoid(pre.double()[:, 3:3 + H] + b.double())
    close(got, gated, DT[dtype], what="gate with bias and constant")
    # the same gate inside the kernel that sums the result into the stream and norms the sum, for all rows and for chosen ones
    gate_rows = pre[:, 3:3 + H].contiguous()
    wb = b.to(w.dtype)
    x2 = resid.float().double() + y.double() * 0.45 * torch.sigmoid(gate_rows.double() + wb.double())
    r3 = resid.float().to(dev)
    out3 = ops.add_rms_norm(r3, y.to(dev), w.to(dev), 1e-5, DT[dtype], groups=groups, gate=(gate_rows.to(dev), wb.to(dev), 0.45))
    close(r3, x2, torch.float32, what="stream after the gated addend")
    close(out3, plain.grouped_norm(x2, w.double(), 1e-5, groups), DT[dtype], what="norm after the gated addend")
    r4 = resid.float().to(dev)
    out4 = ops.add_rms_norm(r4, y.to(dev), w.to(dev), 1e-5, DT[dtype], rows, groups=groups, gate=(gate_rows.to(dev), wb.to(dev), 0.45))
    close(out4, plain.grouped_norm(x2, w.double(), 1e-5, groups)[[T - 1, 0]], DT[dtype], what="norm of chosen rows after the gated addend")
    assert torch.equal(r4.cpu(), resid.float())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d,dv,dims,scaling", [(32, 32, 8, None), (32, 20, 6, dict(factor=8.0, original=64, fast=4.0, slow=1.0)), (32, 16, 0, None),
                                               (48, 48, 20, dict(factor=5.0, original=2048, fast=32.0, slow=1.0)), (64, 64, 64, dict(factor=3.0, original=100, fast=9.0, slow=2.0))])
def test_rotation_with_a_factor_and_normed_values(dtype, d, dv, dims, scaling):
    """``d``: the head size that cache and kernels see; ``dv``: a value head's own size (the rest is padding)."""
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.parts.rotary import RotaryEmbedding
    dev = require_gpu()
    g = torch.Generator().manual_seed(5)
    nq, nkv, P, pages, eps = 6, 2, 8, 5, 2e-3
    pos = [0, 1, 7, 8, 9000, 4095, 33]
    T = len(pos)
    x = rnd(g, T, (nq + 2 * nkv) * d + 17).to(DT[dtype])
    x[:, (nq + nkv) * d:(nq + 2 * nkv) * d].view(T, nkv, d)[:, :, dv:] = 0          # the padding of the value heads
    x[2, (nq + nkv) * d:(nq + 2 * nkv) * d] *= 1e-3                                  # a small value head: eps matters
    freq, mag = None, 1.0
    if dims:
        enc = RotaryEmbedding(d, 20000.0, dims, scaling)
        enc.prepare(dev, 0)
        freq, mag, _ = enc.frequencies()
        pf, pm = plain.ramped_frequencies(dict(base=20000.0, dims=dims, scaling=scaling))
        close(freq, pf, torch.float32, what="frequencies")
        assert abs(mag - pm) < 1e-12 and (scaling is None) == (mag == 1.0)
    kc = torch.full((pages, nkv, P, d), float("nan"), dtype=DT[dtype], device=dev)
    vc = torch.full((pages, nkv, d, P), float("nan"), dtype=DT[dtype], device=dev)
    slots = [3 * P + 1, 0, 4 * P + 7, 9, 2 * P, 17, 30]
    q = ops.bias_rope_store(x.to(dev), nq, nkv, d, None, freq, dims, i32(pos, dev), kc, vc, P, i32(slots, dev), mag=mag, value_norm=(eps, dv))
    f = x.double()[:, :(nq + 2 * nkv) * d]
    rq, rk, rv = f[:, :nq * d].view(T, nq, d), f[:, nq * d:(nq + nkv) * d].view(T, nkv, d), f[:, (nq + nkv) * d:].view(T, nkv, d)
    if dims:
        fr = freq.cpu().double()                     # the kernel's float32 frequencies: what is held here is the rotation
        rq, rk = plain.rotate_half(rq, torch.tensor(pos), fr, mag, dims), plain.rotate_half(rk, torch.tensor(pos), fr, mag, dims)
    rv = torch.cat([plain.rms(rv[..., :dv], eps), rv[..., dv:]], dim=-1)
    tol = 40.0 if dtype == "float32" else 1.0             # float32 angles at position 9000 carry 5e-4 of a radian
    close(q.view(T, nq, d), rq, DT[dtype], scale=tol, what="rotated queries")
    for t, s in enumerate(slots):
        close(kc[s // P, :, s % P, :], rk[t], DT[dtype], scale=tol, what="stored keys")
        close(vc[s // P, :, :, s % P], rv[t], DT[dtype], what="stored values")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nq,nkv,d,dv,dims,cap,T", [(6, 2, 32, 32, 16, 3.0, 150), (4, 4, 64, 80, 64, 8.0, 300), (8, 1, 16, 48, 8, 1.0, 90),
                                                    (3, 1, 12, 10, 4, 2.0, 70), (2, 2, 128, 128, 32, 5.0, 200)])
def test_attention_with_capped_scores_and_normed_values(dtype, nq, nkv, d, dv, dims, cap, T):
    """The attention part on a whole sequence (rows for the large tiles), and the same sequence in portions and single
    tokens with another request beside it (the small tiles over pages), against the plain function.  The scores reach
    several times the cap."""
    from spyinfer_amd.cache import CacheManager
    from spyinfer_amd.cache.storage import CacheStorage
    from spyinfer_amd.parts import PagedAttention, RotaryEmbedding
    from tests.test_gpu_parts import bind, make_batch
    dev = require_gpu()
    W, eps, scale = 72, 1e-5, 0.4
    cfg = dict(heads=nq, kv_heads=nkv, dim=d, vdim=dv, scale=scale, softcap=cap,
               rot=dict(base=30000.0, dims=dims, scaling=dict(factor=4.0, original=64, fast=8.0, slow=1.0)))
    rope = RotaryEmbedding(d, 30000.0, dims, cfg["rot"]["scaling"])
    part = PagedAttention(W, nq, nkv, d, rope, scale=scale, value_dim=dv, names=dict(q=".q", k=".k", v=".v", o=".o"), softcap=cap, value_norm_eps=eps)
    w = bind(part, "a", DT[dtype], dev, 10, 0.35)
    g = torch.Generator().manual_seed(20)
    x = rnd(g, T, W).to(DT[dtype])
    ref = plain.capped_attention(x.double(), {k[2:]: v.double() for k, v in w.items()}, cfg, eps)
    manager = CacheManager([part.cache_spec()], page_size=16, num_pages=2 * (T // 16 + 2), max_num_seqs=3)
    storage = CacheStorage(manager, DT[dtype], dev)
    storage.fill(float("nan"))

    def run(spans, xs):
        batch, entries = make_batch(manager, DT[dtype], dev, spans)
        part.plan(batch)
        batch.upload()
        out = part.forward(torch.cat(xs).to(dev), batch, storage.layer(0))
        for e in entries:
            manager.commit(e.cache, len(e.tokens))
        return out

    a = manager.admit("a")
    # (bfloat16 keys of 128 values under scores of several caps: single elements of early rows, whose softmax has few terms, move by 0.2)
    tol = 3.0 if dtype == "float32" or d < 128 else 12.0
    close(run([(a, T)], [x]), ref, DT[dtype], scale=tol, what="whole")
    manager.release(a)
    a, b = manager.admit("a"), manager.admit("b")
    other = rnd(g, 9, W).to(DT[dtype])
    cut = T - 7
    got = [run([(b, 5), (a, 11)], [other[:5], x[:11]])[5:], run([(a, cut - 11), (b, 1)], [x[11:cut], other[5:6]])[:cut - 11]]
    for t in range(cut, T):
        got.append(run([(b, 1), (a, 1)] if t % 2 else [(a, 1)], [other[6:7], x[t:t + 1]] if t % 2 else [x[t:t + 1]])[-1:])
    close(torch.cat(got), ref, DT[dtype], scale=tol, what="portions and single tokens")
    manager.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,d,dv,taps", [(4, 2, 6, 5, 3), (2, 2, 56, 24, 4), (3, 1, 128, 128, 2), (1, 1, 40, 200, 1), (6, 3, 16, 8, 8)])
def test_delta_rule_with_one_decay_per_head(dtype, H, G, d, dv, taps):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(4)
    lengths, cut, eps = [29, 6, 2], [11, 1, 2], 3e-5
    T, C = sum(lengths), 2 * G * d + H * dv
    raw = rnd(g, T, C + H * dv).to(DT[dtype])                # (rows of a wider product: the gate's columns behind)
    tp = rnd(g, C, taps, std=0.5).to(DT[dtype])
    beta_pre, dec_pre = rnd(g, T, H, std=2.0).float(), rnd(g, T, H, std=2.0).float()
    a_log, dtb, nw = rnd(g, H).to(DT[dtype]), rnd(g, H).to(DT[dtype]), (1.0 + rnd(g, dv, std=0.2)).to(DT[dtype])
    state = torch.full((4, H * d * dv + (taps - 1) * C), float("nan"), device=dev)
    state[[2, 0, 3]] = 0.0
    got = torch.zeros((T, H * dv), dtype=torch.float64)
    for rows, cu, sl, ent in two_steps(lengths, cut):
        x = raw[rows].to(dev)
        qkv = ops.causal_conv_silu(x[:, :C], tp.to(dev), state, H * d * dv, i32(ent, dev), i32(cu, dev), i32(sl, dev))
        y = ops.delta_rule(qkv, beta_pre[rows].to(dev), dec_pre[rows].to(dev), a_log.to(dev), dtb.to(dev), x[:, C:], nw.to(dev), eps,
                           state, i32(cu, dev), i32(sl, dev), H, G, d, dv, gate_act="silu")
        got[rows] = y.double().cpu()
    assert torch.isnan(state[1]).all()
    # the plain function with projections that hand the rows through: identity matrices behind a one-hot input
    h = torch.cat([raw.double(), beta_pre.double(), dec_pre.double()], dim=1)
    eye = torch.eye(h.shape[1], dtype=torch.float64)
    n0 = C + H * dv
    w = {"q": eye[:G * d], "k": eye[G * d:2 * G * d], "v": eye[2 * G * d:C], "g": eye[C:n0], "b": eye[n0:n0 + H], "a": eye[n0 + H:],
         "o": torch.eye(H * dv, dtype=torch.float64), "q.conv": tp.double()[:G * d], "k.conv": tp.double()[G * d:2 * G * d],
         "v.conv": tp.double()[2 * G * d:], "A_log": a_log.double(), "dt_bias": dtb.double(), "norm": nw.double()}
    at = 0
    for L in lengths:
        ref = plain.gated_delta(h[at:at + L], w, dict(heads=H, kv_heads=G, dim=d, vdim=dv), eps)
        close(got[at:at + L], ref, DT[dtype], scale=3.0, what="delta rule %s" % ((H, G, d, dv, taps),))
        at += L


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,d,slow", [(3, 5, False), (2, 40, True), (2, 128, False), (1, 200, True), (4, 64, True), (5, 16, False)])
def test_time_mix_carries_state_and_shifted_row_between_steps(dtype, H, d, slow):
    """``slow``: decays near one, so that what the state took in at a request's start still weighs at its end."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(8)
    lengths, cut, eps = [37, 9, 1, 70], [20, 1, 0, 69], 2e-5
    T, N = sum(lengths), H * d
    r, k, v, gate = (rnd(g, T, N, std=s).to(DT[dtype]) for s in (1.0, d ** -0.5, 1.0, 1.0))
    dec_pre = (rnd(g, T, N) - (4.0 if slow else 0.0)).float()
    w0, u, nw = rnd(g, N, std=0.3).to(DT[dtype]), rnd(g, N, std=0.5).to(DT[dtype]), (1.0 + rnd(g, N, std=0.2)).to(DT[dtype])
    W = N + 3
    x, mu = rnd(g, T, W).to(DT[dtype]), torch.rand((5, W), generator=g, dtype=torch.float64).to(DT[dtype])
    state = torch.full((4, N * d + W), float("nan"), device=dev)
    state[[2, 0, 3, 1]] = 0.0
    got, shifted = torch.zeros((T, N), dtype=torch.float64), torch.zeros((5, T, W), dtype=torch.float64)
    for rows, cu, sl, ent in two_steps(lengths, cut):
        on = lambda t: t[rows].to(dev)
        shifted[:, rows] = ops.token_shift(on(x), mu.to(dev), state, N * d, i32(ent, dev), i32(cu, dev), i32(sl, dev)).double().cpu()
        y = ops.time_mix(on(r), on(k), on(v), on(dec_pre), w0.to(dev), u.to(dev), on(gate), nw.to(dev), eps, state, i32(cu, dev), i32(sl, dev), H, d)
        got[rows] = y.double().cpu()
    # the plain function with projections that hand the rows through (blends of zero: every projection reads its own
    # columns of the token itself); the tanh between the decay's two projections sees numbers so small that it is the identity
    h = torch.cat([t.double() for t in (r, k, v, gate, dec_pre)], dim=1)
    eye = torch.eye(5 * N, dtype=torch.float64)
    w = {"mu." + s: torch.zeros(5 * N, dtype=torch.float64) for s in "rkvgw"}
    w.update({"r": eye[:N], "k": eye[N:2 * N], "v": eye[2 * N:3 * N], "g": eye[3 * N:4 * N], "w1": eye[4 * N:] * 1e-5,
              "w2": torch.eye(N, dtype=torch.float64) * 1e5, "w0": w0.double(), "u": u.double().view(H, d), "norm": nw.double(),
              "o": torch.eye(N, dtype=torch.float64)})
    at = 0
    for L in lengths:
        ref = plain.time_mix(h[at:at + L], w, dict(heads=H, dim=d), eps)
        close(got[at:at + L], ref, DT[dtype], scale=3.0, what="time mix %s" % ((H, d),))
        xs = x.double()[at:at + L]
        prev = torch.cat([torch.zeros((1, W), dtype=torch.float64), xs[:-1]])
        close(shifted[:, at:at + L], xs[None] + (prev - xs)[None] * mu.double()[:, None, :], DT[dtype], what="token shift")
        at += L


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,W", [(7, 40), (3, 4096), (130, 192)])
def test_two_results_normed_and_averaged(dtype, T, W):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(9)
    a, b = rnd(g, T, W, std=5.0).to(DT[dtype]), rnd(g, T, W, std=0.02).to(DT[dtype])
    wa, wb = (1.0 + rnd(g, W, std=0.3)).to(DT[dtype]), (1.0 + rnd(g, W, std=0.3)).to(DT[dtype])
    got = ops.norm_pair_mean(a.to(dev), b.to(dev), wa.to(dev), wb.to(dev), 1e-4)
    ref = 0.5 * (plain.rms(a.double(), 1e-4) * wa.double() + plain.rms(b.double(), 1e-4) * wb.double())
    close(got, ref, DT[dtype], what="normed pair")


@pytest.mark.parametrize("E,top", [(12, 3), (8, 1), (1, 1), (64, 8), (6, 6), (130, 5)])
def test_router_with_sigmoid_scores_as_they_are(E, top):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(6)
    T = 50
    z = rnd(g, T, E, std=2.0).float()
    ids, w = ops.moe_route(z.to(dev), None, top, 1, 1, 1.0, score="sigmoid", renormalize=False)
    rid, rw = plain.sigmoid_route(z.double(), top)
    for t in range(T):
        got = sorted(zip(ids[t].tolist(), w[t].tolist()))
        ref = sorted(zip(rid[t].tolist(), rw[t].tolist()))
        assert [e for e, _ in got] == [e for e, _ in ref], "token %d: experts %r, expected %r" % (t, got, ref)
        assert all(abs(a - b) < 1e-5 for (_, a), (_, b) in zip(got, ref))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,K,F,E,top", [(1, 48, 24, 8, 3), (37, 64, 40, 6, 2), (300, 128, 96, 12, 4), (5, 40, 8, 4, 4), (64, 256, 128, 130, 5),
                                         (200, 1288, 72, 4, 2), (6, 1288, 48, 8, 2), (90, 192, 64, 16, 1)])
def test_experts_with_weighted_inputs_and_clamps(dtype, T, K, F, E, top):
    """Inputs large enough that all three clamps bite; the weight must enter ahead of them."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(7)
    limit = 1.25
    x = rnd(g, T, K, std=2.0).to(DT[dtype])
    wgu, wd = rnd(g, E, 2 * F, K, std=K ** -0.5).to(DT[dtype]), rnd(g, E, K, F, std=F ** -0.5).to(DT[dtype])
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    if T > 20:
        ids[:20] = torch.arange(top, dtype=torch.int32)          # one expert with many rows, others with none
    w = torch.rand((T, top), generator=g)
    out = ops.moe_experts(x.to(dev), ids.to(dev), w.to(dev), wgu.to(dev), wd.to(dev), activation="clamped", limit=limit, weight_input=True)
    ref = torch.zeros((T, K), dtype=torch.float64)
    clamped = 0
    for t in range(T):
        for j in range(top):
            e = int(ids[t, j])
            xin = w[t, j].double() * x[t:t + 1].double()
            clamped += int(((xin @ wgu[e, :F].double().T) > limit).sum()) + int(((xin @ wgu[e, F:].double().T).abs() > limit).sum())
            ref[t] += plain.clamped_expert(xin, wgu[e, :F].double(), wgu[e, F:].double(), wd[e].double(), limit)[0]
    assert clamped > 0
    close(out, ref, DT[dtype], scale=3.0, what="experts")


# ---- whole models ------------------------------------------------------------------------------
MODELS = {"odd": (mc.MER_ODD, 2, None), "a": (mc.MER_A, 3, None), "b": (mc.MER_B, 4, None), "c": (mc.MER_C, 6, mc.decisive_router()), "a_sharp": (mc.MER_A, 5, mc.sharpen()),
          "a_memory": (mc.MER_A, 9, mc.long_memory()), "c_memory": (mc.MER_C, 11, mc.both(mc.long_memory(w0=-3.0), mc.decisive_router())),
          "far_sharp": (mc.MER_FAR, 8, mc.both(mc.sharpen(8.0), mc.long_memory())), "c_sharp": (mc.MER_C, 12, mc.both(mc.sharpen(3.0), mc.long_memory()))}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: mc.write_model(str(tmp_path_factory.mktemp("gmer_" + name)), cfg, seed, tweak) for name, (cfg, seed, tweak) in MODELS.items()}


# (sharpened scores carry several times the rounding of a bfloat16 key: those models are held in float32 only)
@pytest.mark.parametrize("name,dtype", [(n, d) for n in ("a", "b", "c", "odd", "a_sharp", "a_memory", "c_memory") for d in ("float32", "bfloat16")
                                        if not (n.endswith("sharp") and d == "bfloat16")])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_schedules_equal_the_plain_implementation(folders, name, mode, dtype, tmp_path):
    require_gpu()
    folder = folders[name]
    requests = rc.random_requests(mc.vocab_of(folder), [41, 1, 2, 130, 23, 30, 52, 38, 75], 7)
    steps = {"whole": rc.whole, "bulk_tail": lambda r: rc.bulk_tail(r, 40), "portions": rc.portions, "mixed": rc.mixed}[mode](requests)
    rc.run_replay_inprocess(folder, dtype, str(tmp_path), steps, rc.max_live_tokens(steps),
                            ["--kvcache-block-size", "8" if not name.startswith("c") else "16", "--poison-cache"])
    compare(rc.collect(str(tmp_path), steps, mc.vocab_of(folder)), mc.plain_logits(folder, requests), dtype, "%s/%s/%s" % (name, mode, dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recurrences_alone_run_without_any_page_group(dtype, tmp_path):
    require_gpu()
    folder = mc.write_model(str(tmp_path / "m"), mc.MER_REC, 1, None)
    requests = rc.random_requests(53, [21, 1, 2, 33, 9], 5)
    ref = mc.plain_logits(folder, requests)
    for name, steps in (("whole", rc.whole(requests)), ("portions", rc.portions(requests)), ("mixed", rc.mixed(requests))):
        out = str(tmp_path / name)
        rc.run_replay_inprocess(folder, dtype, out, steps, rc.max_live_tokens(steps), ["--poison-cache"])
        compare(rc.collect(out, steps, 53), ref, dtype, "recurrences alone/%s/%s" % (name, dtype))


@pytest.mark.parametrize("name", ["far_sharp", "c_sharp"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_far_keys_and_old_state_among_hundreds_of_tokens(folders, name, mode, tmp_path):
    """Sharp scores: the keys that decide a row's result lie anywhere in 600 tokens, across many pages; recurrences that
    forget slowly: what the states took in at a request's start still weighs at its end."""
    require_gpu()
    folder = folders[name]
    requests = rc.random_requests(mc.vocab_of(folder), [600, 333, 2, 150], 12)
    steps = {"whole": rc.whole, "bulk_tail": lambda r: rc.bulk_tail(r, 50), "portions": lambda r: rc.portions(r, (100, 3, 2, 257, 64, 1)),
             "mixed": lambda r: rc.mixed(r, seed=3)}[mode](requests)
    rc.run_replay_inprocess(folder, "float32", str(tmp_path), steps, rc.max_live_tokens(steps), ["--poison-cache"])
    rc.compare(rc.collect(str(tmp_path), steps, mc.vocab_of(folder)), mc.plain_logits(folder, requests), what="far/" + mode, **TOL["float32"])


@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions"])
def test_long_requests_in_bfloat16_on_the_matrix_cores(folders, mode, tmp_path):
    """Portions of hundreds of tokens take the attention's large tiles, single tokens over hundreds of keys its small
    ones, both with capped scores; the experts' products take their kernels for many rows."""
    require_gpu()
    folder = folders["c_memory"]
    requests = rc.random_requests(400, [700, 260], 21)
    steps = {"whole": rc.whole, "bulk_tail": lambda r: rc.bulk_tail(r, 60), "portions": lambda r: rc.portions(r, (300, 2, 129, 64, 5, 411, 33))}[mode](requests)
    rc.run_replay_inprocess(folder, "bfloat16", str(tmp_path), steps, rc.max_live_tokens(steps), ["--poison-cache"])
    compare(rc.collect(str(tmp_path), steps, 400), mc.plain_logits(folder, requests), "bfloat16", "long/%s" % mode)


def test_long_decoding(folders, tmp_path):
    require_gpu()
    folder = folders["a_memory"]
    requests = rc.random_requests(97, [260], 13)
    steps = rc.bulk_tail(requests, 250)
    rc.run_replay_inprocess(folder, "float32", str(tmp_path), steps, rc.max_live_tokens(steps), ["--kvcache-block-size", "8", "--poison-cache"])
    rc.compare(rc.collect(str(tmp_path), steps, 97), mc.plain_logits(folder, requests), what="long decoding", **TOL["float32"])


# ---- the entry point ---------------------------------------------------------------------------
@pytest.mark.parametrize("eager", [True, False])
def test_greedy_generation_equals_plain(folders, eager):
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    require_gpu()
    folder = folders["a"]
    model = plain.PlainMeronex.from_folder(folder)
    prompts = list(rc.random_requests(97, [5, 17, 2, 30, 9], 9).values())
    want = [model.greedy(p, 24) for p in prompts]
    for opts in (dict(), dict(max_num_batched_tokens=12, prefill_chunk=7, max_num_seqs=2)):
        kw = dict(dtype="float32", max_model_len=64, num_kvcache_blocks=24, max_num_seqs=4, kvcache_block_size=8, enforce_eager=eager)
        kw.update(opts)
        eng = LLMEngine(folder, **kw)
        assert eng.generate(prompts, SamplingParams(max_new_tokens=24, ignore_eos=True)) == want
        if not eager:
            assert eng.runner.graph_replays > 0
        eng.runner.manager.check()


def test_bfloat16_generation_follows_the_plain_logits(folders):
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    require_gpu()
    folder = folders["c"]
    model = plain.PlainMeronex.from_folder(folder)
    prompts = list(rc.random_requests(400, [33, 70, 8], 10).values())
    eng = LLMEngine(folder, dtype="bfloat16", max_model_len=128, num_kvcache_blocks=40, max_num_seqs=4, enforce_eager=False)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=12, ignore_eos=True))
    for p, out in zip(prompts, outs):
        toks = list(p)
        for t in out:
            logits = model.forward(toks)[-1]
            best = int(torch.argmax(logits))
            near = 0.2 + 0.15 * float(logits.pow(2).mean().sqrt())
            assert t == best or float(logits[best] - logits[t]) < near, "token %d where the plain logits prefer %d clearly" % (t, best)
            toks.append(t)


def test_trace_run_as_a_program(folders, tmp_path):
    require_gpu()
    folder = folders["b"]
    requests = rc.random_requests(61, [19, 40], 14)
    steps = rc.portions(requests)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(tmp_path),
                        "--max-tokens", str(rc.max_live_tokens(steps))], input="".join(json.dumps(s) + "\n" for s in steps),
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    rc.compare(rc.collect(str(tmp_path), steps, 61), mc.plain_logits(folder, requests), what="trace_run", **TOL["float32"])


def test_command_line_generates(folders):
    require_gpu()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-m", "spyinfer_amd", "-m", folders["a"], "--dtype", "float32", "--random-prompts", "5,9",
                        "--max-new-tokens", "6", "--max-model-len", "64", "--num-kvcache-blocks", "16", "--max-num-seqs", "4"],
                       cwd=root, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert r.stdout.strip(), "the command line printed no tokens"
