"""Sodedra on the GPU: every mechanism's kernel against the plain implementation's function, then whole models through
the trace replay (the engine's step function, cache manager and kernels) under every schedule, long decoding, and
greedy generation through the entry point with and without captured steps."""
import json
import os
import subprocess
import sys

import pytest
import torch

from tests import replay_cases as rc
from tests import sodedra_cases as sc
from tests.gpu_util import close, require_gpu
from tests.plain import sodedra_plain as plain

pytestmark = pytest.mark.gpu
TOL = {"float32": dict(atol=3e-4, rtol=3e-4), "bfloat16": dict(atol=1.5e-1, rtol=4e-2)}
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def compare(got, ref, dtype, what):
    """float32: every logit within a small tolerance.  bfloat16: a row's error, root mean square over the vocabulary,
    against the row's own root mean square, for nine rows in ten and in the median.  Single rows may be far off in
    bfloat16 although nothing is wrong: a router's close call picks another expert, and a matrix memory's first
    read-outs divide by n . q, which rounding can move across zero; float32 holds every row."""
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
    assert float(rel.median()) < 0.03 and float(rel.quantile(0.9)) < 0.06, \
        "%s: rows are off by %.3f of their size in the median, %.3f at the ninth decile" % (what, float(rel.median()), float(rel.quantile(0.9)))


def i32(values, dev):
    return torch.tensor(values, dtype=torch.int32, device=dev)


def rnd(g, *shape, std=1.0):
    return torch.randn(shape, generator=g, dtype=torch.float64) * std


def two_steps(lengths, cut):
    """Two steps over requests of ``lengths`` tokens in slots 2, 0, 3, ...: the first ``cut[i]`` tokens, then the rest, the
    entries in another order.  Yields (rows of the flattened sequences, cu_q, slot ids, token_entry)."""
    slots = [2, 0, 3, 1][:len(lengths)]
    first = [0]
    for n in lengths:
        first.append(first[-1] + n)
    for order, part in ((range(len(lengths)), 0), (reversed(range(len(lengths))), 1)):
        rows, cu, sl, ent = [], [0], [], []
        for i in order:
            lo, hi = (0, cut[i]) if part == 0 else (cut[i], lengths[i])
            if hi > lo:
                ent += [len(sl)] * (hi - lo)
                rows += list(range(first[i] + lo, first[i] + hi))
                cu.append(len(rows))
                sl.append(slots[i])
        yield rows, cu, sl, ent


# ---- mechanisms --------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,H", [(13, 50), (5, 2048), (70, 1100)])
def test_norm_with_two_addends_and_scaled_embedding(dtype, T, H):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(2)
    resid, a, b, w = rnd(g, T, H), rnd(g, T, H).to(DT[dtype]), rnd(g, T, H).to(DT[dtype]), rnd(g, H, std=0.3)
    r = resid.float().to(dev)
    out = ops.add_rms_norm(r, a.to(dev), (1.0 + w).float().to(dev), 1e-5, DT[dtype], delta2=b.to(dev))
    x = resid.float().double() + (a.double() + b.double())
    close(r, x, torch.float32, what="stream after two addends")
    close(out, plain.zero_centred_norm(x, w.float().double(), 1e-5), DT[dtype], what="norm after two addends")
    rows = i32([T - 1, 0], dev)
    r2 = resid.float().to(dev)
    out2 = ops.add_rms_norm(r2, a.to(dev), (1.0 + w).float().to(dev), 1e-5, DT[dtype], rows, delta2=b.to(dev))
    close(out2, plain.zero_centred_norm(x, w.float().double(), 1e-5)[[T - 1, 0]], DT[dtype], what="norm of chosen rows")
    assert torch.equal(r2.cpu(), resid.float())
    table = rnd(g, 31, H).to(DT[dtype])
    ids = torch.randint(0, 31, (T,), generator=g)
    close(ops.embedding(i32(ids.tolist(), dev), table.to(dev), 0.37), table.double()[ids] * 0.37, torch.float32, what="scaled embedding")


def scan_pieces(cu, piece):
    """The pieces of a step's entries as the engine plans them: int32 [4 n] and whether an entry has several."""
    rec = [(e, t, min(t + piece, cu[e + 1])) for e in range(len(cu) - 1) for t in range(cu[e], cu[e + 1], piece)]
    first = [min(k for k, r in enumerate(rec) if r[0] == e) for e, _, _ in rec]
    return [r[0] for r in rec] + [r[1] for r in rec] + [r[2] for r in rec] + first, len(rec), len(rec) > len(cu) - 1


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("lengths,cut,piece", [([37, 9, 1], [20, 1, 0], 0), ([150, 70, 1], [100, 64, 0], 64), ([37, 9, 2], [20, 1, 1], 4)])
@pytest.mark.parametrize("H,d,dv", [(3, 5, 7), (2, 40, 72), (2, 128, 96), (1, 200, 300), (2, 64, 600)])
def test_mlstm_carries_its_state_between_steps(dtype, H, d, dv, lengths, cut, piece):
    """``piece`` > 0: entries are cut into pieces of that many tokens, walked by different waves and composed."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(3)
    cap, eps = 6.0, 2e-5
    T = sum(lengths)
    proj = rnd(g, T, 2 * H * d + 2 * H * dv).to(DT[dtype])
    gates = rnd(g, T, 2 * H, std=3.0).float()
    bi, bf, nw = rnd(g, H).to(DT[dtype]), (rnd(g, H) + 2.0).to(DT[dtype]), (1.0 + rnd(g, H * dv, std=0.2)).to(DT[dtype])
    state = torch.full((4, ops.mlstm_state_size(H, d, dv)), float("nan"), device=dev)
    state[[2, 0, 3]] = 0.0
    got = torch.zeros((T, H * dv), dtype=torch.float64)
    for rows, cu, sl, _ in two_steps(lengths, cut):
        pieces = None
        if piece:
            arr, n, multi = scan_pieces(cu, piece)
            pieces = (i32(arr, dev), n, multi)
        y = ops.mlstm(proj[rows].to(dev), 0, H * d, 2 * H * d, 2 * H * d + H * dv, gates[rows].to(dev), bi.to(dev), bf.to(dev), cap,
                      nw.to(dev), eps, state, i32(cu, dev), i32(sl, dev), H, d, dv, pieces=pieces)
        got[rows] = y.double().cpu()
    assert torch.isnan(state[1]).all()
    # the plain function with projections that hand the rows through: identity matrices behind a one-hot input
    p = proj.double()
    eye = torch.eye(p.shape[1] + 2 * H, dtype=torch.float64)
    h = torch.cat([p, gates.double()], dim=1)
    n = 2 * H * d + 2 * H * dv
    w = {"q": eye[:H * d], "k": eye[H * d:2 * H * d], "v": eye[2 * H * d:2 * H * d + H * dv], "g": eye[2 * H * d + H * dv:n],
         "i": eye[n:n + H], "f": eye[n + H:], "i.b": bi.double(), "f.b": bf.double(), "norm": nw.double(), "o": torch.eye(H * dv, dtype=torch.float64)}
    at = 0
    for L in lengths:
        ref = plain.mlstm(h[at:at + L], w, dict(heads=H, dim=d, vdim=dv, gate_cap=cap), eps)
        close(got[at:at + L], ref, DT[dtype], what="mlstm %s" % ((H, d, dv),))
        at += L


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,G,d,dv,taps", [(4, 2, 6, 5, 3), (2, 2, 56, 24, 4), (3, 1, 128, 128, 2), (1, 1, 40, 200, 1), (2, 1, 16, 8, 8)])
def test_delta_rule_and_convolution_carry_their_state_between_steps(dtype, H, G, d, dv, taps):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(4)
    lengths, cut, eps = [29, 6, 2], [11, 1, 2], 3e-5
    T, C = sum(lengths), 2 * G * d + H * dv
    raw = rnd(g, T, C + 3).to(DT[dtype])                     # (rows of a wider product: three more columns behind)
    tp = rnd(g, C, taps, std=0.5).to(DT[dtype])
    beta_pre, dec_pre = rnd(g, T, H, std=2.0).float(), rnd(g, T, H * d, std=2.0).float()
    a_log, dtb, nw = rnd(g, H).to(DT[dtype]), rnd(g, H * d).to(DT[dtype]), (1.0 + rnd(g, dv, std=0.2)).to(DT[dtype])
    gate = rnd(g, T, H * dv).to(DT[dtype])
    state = torch.full((4, H * d * dv + (taps - 1) * C), float("nan"), device=dev)
    state[[2, 0, 3]] = 0.0
    got = torch.zeros((T, H * dv), dtype=torch.float64)
    conv = torch.zeros((T, C), dtype=torch.float64)
    for rows, cu, sl, ent in two_steps(lengths, cut):
        x = raw[rows].to(dev)
        qkv = ops.causal_conv_silu(x[:, :C], tp.to(dev), state, H * d * dv, i32(ent, dev), i32(cu, dev), i32(sl, dev))
        conv[rows] = qkv.double().cpu()
        y = ops.delta_rule(qkv, beta_pre[rows].to(dev), dec_pre[rows].to(dev), a_log.to(dev), dtb.to(dev), gate[rows].to(dev), nw.to(dev), eps,
                           state, i32(cu, dev), i32(sl, dev), H, G, d, dv)
        got[rows] = y.double().cpu()
    assert torch.isnan(state[1]).all()
    p = raw.double()[:, :C]
    h = torch.cat([p, beta_pre.double(), dec_pre.double(), gate.double()], dim=1)
    eye = torch.eye(h.shape[1], dtype=torch.float64)
    n0, n1, n2 = C, C + H, C + H + H * d
    w = {"q": eye[:G * d], "k": eye[G * d:2 * G * d], "v": eye[2 * G * d:C], "b": eye[n0:n1], "a1": eye[n1:n2], "a2": torch.eye(H * d, dtype=torch.float64),
         "g1": eye[n2:], "g2": torch.eye(H * dv, dtype=torch.float64), "o": torch.eye(H * dv, dtype=torch.float64),
         "q.conv": tp.double()[:G * d], "k.conv": tp.double()[G * d:2 * G * d], "v.conv": tp.double()[2 * G * d:],
         "A_log": a_log.double(), "dt_bias": dtb.double(), "norm": nw.double()}
    at = 0
    for L in lengths:
        close(conv[at:at + L], plain.silu(plain.causal_conv(p[at:at + L], tp.double())), DT[dtype], what="convolution")
        ref = plain.channel_delta(h[at:at + L], w, dict(heads=H, kv_heads=G, dim=d, vdim=dv), eps)
        close(got[at:at + L], ref, DT[dtype], scale=3.0, what="delta rule %s" % ((H, G, d, dv, taps),))
        at += L


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("dims,scaling", [(8, None), (6, dict(factor=8.0, low=1.0, high=4.0, original=64)), (0, None), (20, dict(factor=5.0, low=1.0, high=3.0, original=2048))])
def test_biases_rotation_and_store(dtype, dims, scaling):
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.parts.rotary import RotaryEmbedding
    dev = require_gpu()
    g = torch.Generator().manual_seed(5)
    nq, nkv, d, P, pages = 6, 2, 32, 8, 5
    pos = [0, 1, 7, 8, 9000, 4095, 33]
    T = len(pos)
    x = rnd(g, T, (nq + 2 * nkv) * d + 17).to(DT[dtype])
    bias = rnd(g, (nq + 2 * nkv) * d).to(DT[dtype])
    freq = None
    if dims:
        enc = RotaryEmbedding(d, 20000.0, dims, scaling)
        enc.prepare(dev, 0)
        freq = enc.frequencies()[0]
        close(freq, plain.scaled_frequencies(dims, 20000.0, scaling), torch.float32, what="frequencies")
    kc = torch.full((pages, nkv, P, d), float("nan"), dtype=DT[dtype], device=dev)
    vc = torch.full((pages, nkv, d, P), float("nan"), dtype=DT[dtype], device=dev)
    slots = [3 * P + 1, 0, 4 * P + 7, 9, 2 * P, 17, 30]
    q = ops.bias_rope_store(x.to(dev), nq, nkv, d, bias.to(dev), freq, dims, i32(pos, dev), kc, vc, P, i32(slots, dev))
    f = x.double()[:, :(nq + 2 * nkv) * d] + bias.double()
    rq, rk, rv = f[:, :nq * d].view(T, nq, d), f[:, nq * d:(nq + nkv) * d].view(T, nkv, d), f[:, (nq + nkv) * d:].view(T, nkv, d)
    if dims:
        fr = freq.cpu().double()                     # the kernel's float32 frequencies: what is held here is the rotation
        rq, rk = plain.rotate_half(rq, torch.tensor(pos), fr, dims), plain.rotate_half(rk, torch.tensor(pos), fr, dims)
    tol = 40.0 if dtype == "float32" else 1.0             # float32 angles at position 9000 carry 5e-4 of a radian
    close(q.view(T, nq, d), rq, DT[dtype], scale=tol, what="rotated queries")
    for t, s in enumerate(slots):
        close(kc[s // P, :, s % P, :], rk[t], DT[dtype], scale=tol, what="stored keys")
        close(vc[s // P, :, :, s % P], rv[t], DT[dtype], what="stored values")
    y = rnd(g, T, 24).to(DT[dtype])
    wide = rnd(g, T, 40).to(DT[dtype])
    close(ops.sigmoid_gate(y.to(dev), wide.to(dev)[:, 9:33]), y.double() * torch.sigmoid(wide.double()[:, 9:33]), DT[dtype], what="gate")


@pytest.mark.parametrize("E,top,groups,keep", [(12, 3, 3, 2), (8, 3, 4, 2), (4, 1, 1, 1), (64, 8, 8, 4), (6, 6, 3, 3), (130, 5, 10, 2)])
def test_router_chooses_among_the_best_groups(E, top, groups, keep):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(6)
    T = 50
    z = rnd(g, T, E, std=2.0).float()
    corr = rnd(g, E, std=0.3).float() - 0.4          # choice scores may be negative: a barred expert counts as minus infinity, not 0
    ids, w = ops.moe_route(z.to(dev), corr.to(dev), top, groups, keep, 1.7)
    rid, rw = plain.route(z.double(), corr.double(), top, groups, keep, 1.7)
    for t in range(T):
        got = sorted(zip(ids[t].tolist(), w[t].tolist()))
        ref = sorted(zip(rid[t].tolist(), rw[t].tolist()))
        assert [e for e, _ in got] == [e for e, _ in ref], "token %d: experts %r, expected %r" % (t, got, ref)
        assert all(abs(a - b) < 1e-5 for (_, a), (_, b) in zip(got, ref))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,K,F,E,top", [(1, 48, 24, 8, 3), (37, 64, 40, 6, 2), (300, 128, 96, 12, 4), (5, 40, 8, 4, 4), (64, 256, 128, 130, 5),
                                         (200, 1288, 72, 4, 2), (6, 1288, 48, 8, 2)])      # (many steps of K, the last one in part)
def test_experts_over_sorted_pairs(dtype, T, K, F, E, top):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(7)
    x = rnd(g, T, K).to(DT[dtype])
    wgu, wd = rnd(g, E, 2 * F, K, std=K ** -0.5).to(DT[dtype]), rnd(g, E, K, F, std=F ** -0.5).to(DT[dtype])
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    if T > 20:
        ids[:20] = torch.arange(top, dtype=torch.int32)          # one expert with many rows, others with none
    w = torch.rand((T, top), generator=g)
    out = ops.moe_experts(x.to(dev), ids.to(dev), w.to(dev), wgu.to(dev), wd.to(dev))
    ref = torch.zeros((T, K), dtype=torch.float64)
    for t in range(T):
        for j in range(top):
            e = int(ids[t, j])
            ref[t] += w[t, j].double() * plain.gated_ff(x[t:t + 1].double(), wgu[e, :F].double(), wgu[e, F:].double(), wd[e].double())[0]
    close(out, ref, DT[dtype], scale=2.0, what="experts")


# ---- whole models ------------------------------------------------------------------------------
MODELS = {"a": (sc.SOD_A, 3, None), "b": (sc.SOD_B, 4, None), "c": (sc.SOD_C, 6, None), "a_sharp": (sc.SOD_A, 5, sc.sharpen()),
          "a_memory": (sc.SOD_A, 9, sc.long_memory()), "c_router": (sc.SOD_C, 11, sc.biased_router()),
          "long_sharp": (sc.SOD_LONG, 7, lambda t: (sc.sharpen(5.0)(t), sc.long_memory()(t))), "long_memory": (sc.SOD_LONG, 7, sc.long_memory()),
          "far_sharp": (sc.SOD_FAR, 8, sc.sharpen(8.0))}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: sc.write_model(str(tmp_path_factory.mktemp("gsod_" + name)), cfg, seed, tweak) for name, (cfg, seed, tweak) in MODELS.items()}


# (scores sharpened sixfold carry six times the rounding of a bfloat16 key: those models are held in float32 only)
@pytest.mark.parametrize("name,dtype", [(n, d) for n in ("a", "b", "c", "a_sharp", "a_memory", "c_router") for d in ("float32", "bfloat16")
                                        if not (n.endswith("sharp") and d == "bfloat16")])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_schedules_equal_the_plain_implementation(folders, name, mode, dtype, tmp_path):
    require_gpu()
    folder = folders[name]
    requests = rc.random_requests(sc.vocab_of(folder), [41, 1, 2, 130, 23, 30, 52, 38, 75], 7)
    steps = {"whole": rc.whole, "bulk_tail": lambda r: rc.bulk_tail(r, 40), "portions": rc.portions, "mixed": rc.mixed}[mode](requests)
    rc.run_replay_inprocess(folder, dtype, str(tmp_path), steps, rc.max_live_tokens(steps),
                            ["--kvcache-block-size", "8" if not name.startswith("c") else "16", "--poison-cache"])
    compare(rc.collect(str(tmp_path), steps, sc.vocab_of(folder)), sc.plain_logits(folder, requests), dtype, "%s/%s/%s" % (name, mode, dtype))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recurrences_alone_run_without_any_page_group(dtype, tmp_path):
    require_gpu()
    folder = sc.write_model(str(tmp_path / "m"), sc.SOD_REC, 1, None)
    requests = rc.random_requests(53, [21, 1, 2, 33, 9], 5)
    ref = sc.plain_logits(folder, requests)
    for name, steps in (("whole", rc.whole(requests)), ("portions", rc.portions(requests)), ("mixed", rc.mixed(requests))):
        out = str(tmp_path / name)
        rc.run_replay_inprocess(folder, dtype, out, steps, rc.max_live_tokens(steps), ["--poison-cache"])
        compare(rc.collect(out, steps, 53), ref, dtype, "recurrences alone/%s/%s" % (name, dtype))


@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions"])
def test_far_keys_among_hundreds(folders, mode, tmp_path):
    """One attention layer without a window and with sharp scores: the keys that decide a row's result lie anywhere in
    600 tokens, across many pages."""
    require_gpu()
    folder = folders["far_sharp"]
    requests = rc.random_requests(sc.vocab_of(folder), [600, 333], 12)
    steps = {"whole": rc.whole, "bulk_tail": lambda r: rc.bulk_tail(r, 50), "portions": lambda r: rc.portions(r, (100, 3, 2, 257, 64, 1))}[mode](requests)
    rc.run_replay_inprocess(folder, "float32", str(tmp_path), steps, rc.max_live_tokens(steps), ["--poison-cache"])
    rc.compare(rc.collect(str(tmp_path), steps, sc.vocab_of(folder)), sc.plain_logits(folder, requests), what="far/" + mode, **TOL["float32"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_long_requests_under_windows_of_hundreds(folders, mode, dtype, tmp_path):
    """Requests of up to 900 tokens, windows of 333 and 150 tokens, sharp scores, recurrences that forget slowly;
    decoding passes the windows' edges over prompt tokens and decoded ones; four such requests share pages and slots in
    the mixed schedule."""
    require_gpu()
    folder = folders["long_sharp" if dtype == "float32" else "long_memory"]
    requests = rc.random_requests(211, [900, 400, 700, 3, 520], 21)
    steps = {"whole": rc.whole, "bulk_tail": lambda r: rc.bulk_tail(r, 200), "portions": lambda r: rc.portions(r, (300, 2, 129, 64, 5, 411, 33)),
             "mixed": lambda r: rc.mixed(r, seed=3)}[mode](requests)
    rc.run_replay_inprocess(folder, dtype, str(tmp_path), steps, rc.max_live_tokens(steps), ["--poison-cache"])
    compare(rc.collect(str(tmp_path), steps, 211), sc.plain_logits(folder, requests), dtype, "long/%s/%s" % (mode, dtype))


def test_long_decoding_passes_many_windows(folders, tmp_path):
    require_gpu()
    folder = folders["a_memory"]
    requests = rc.random_requests(97, [260], 13)
    steps = rc.bulk_tail(requests, 250)
    rc.run_replay_inprocess(folder, "float32", str(tmp_path), steps, rc.max_live_tokens(steps), ["--kvcache-block-size", "8", "--poison-cache"])
    rc.compare(rc.collect(str(tmp_path), steps, 97), sc.plain_logits(folder, requests), what="long decoding", **TOL["float32"])


# ---- the entry point ---------------------------------------------------------------------------
@pytest.mark.parametrize("eager", [True, False])
def test_greedy_generation_equals_plain(folders, eager):
    from spyinfer_amd.engine.llm_engine import LLMEngine
    from spyinfer_amd.sampling import SamplingParams
    require_gpu()
    folder = folders["a"]
    model = plain.PlainSodedra.from_folder(folder)
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
    model = plain.PlainSodedra.from_folder(folder)
    prompts = list(rc.random_requests(400, [33, 70, 8], 10).values())
    eng = LLMEngine(folder, dtype="bfloat16", max_model_len=128, num_kvcache_blocks=40, max_num_seqs=4, enforce_eager=False)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=12, ignore_eos=True))
    for p, out in zip(prompts, outs):
        toks = list(p)
        for t in out:
            logits = model.forward(toks)[-1]
            best = int(torch.argmax(logits))
            assert t == best or float(logits[best] - logits[t]) < 0.2, "token %d where the plain logits prefer %d clearly" % (t, best)
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
    rc.compare(rc.collect(str(tmp_path), steps, 61), sc.plain_logits(folder, requests), what="trace_run", **TOL["float32"])


def test_command_line_generates(folders):
    require_gpu()
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-m", "spyinfer_amd", "-m", folders["a"], "--dtype", "float32", "--random-prompts", "5,9",
                        "--max-new-tokens", "6", "--max-model-len", "64", "--num-kvcache-blocks", "16", "--max-num-seqs", "4"],
                       cwd=root, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert r.stdout.strip(), "the command line printed no tokens"
