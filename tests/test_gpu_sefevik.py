"""Sefevik on the GPU: every mechanism's kernel against the plain implementation's function, then whole models through
the trace replay (the engine's step function, cache manager and kernels) under every schedule, long decoding, and
greedy generation through the entry point with and without captured steps."""
import os
import subprocess
import sys

import pytest
import torch

from tests import replay_cases as rc
from tests import sefevik_cases as sc
from tests.gpu_util import close, require_gpu
from tests.plain import sefevik_plain as plain

pytestmark = pytest.mark.gpu
TOL = {"float32": dict(atol=2e-4, rtol=2e-4), "bfloat16": dict(atol=1e-1, rtol=3e-2)}
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def i32(values, dev):
    return torch.tensor(values, dtype=torch.int32, device=dev)


# ---- mechanisms --------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pair_embedding_keeps_the_previous_token_in_the_slot(dtype):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(1)
    V, H, buckets, mp, mc = 37, 24, 11, 5, 3
    table = torch.randn((V, H), generator=g).to(DT[dtype])
    pair = torch.randn((buckets + 1, H), generator=g).to(DT[dtype])
    seqs = {2: torch.randint(0, V, (9,), generator=g).tolist(), 0: torch.randint(0, V, (4,), generator=g).tolist()}
    last = torch.full((3,), -7, dtype=torch.int32, device=dev)
    got = {s: [] for s in seqs}
    # step 1: 5 tokens of slot 2 and 1 of slot 0; step 2: the rest (the entries' first tokens read the slots)
    for cuts in ({2: (0, 5), 0: (0, 1)}, {0: (1, 4), 2: (5, 9)}):
        ids, pos, ent, cu, slots = [], [], [], [0], []
        for e, (s, (lo, hi)) in enumerate(cuts.items()):
            ids += seqs[s][lo:hi]; pos += list(range(lo, hi)); ent += [e] * (hi - lo); cu.append(len(ids)); slots.append(s)
        out, copy = ops.pair_embedding(i32(ids, dev), table.to(dev), pair.to(dev), buckets, mp, mc, i32(pos, dev), i32(ent, dev),
                                       i32(cu, dev), i32(slots, dev), last, DT[dtype])
        assert (copy is None) == (dtype == "float32")
        for e, s in enumerate(cuts):
            got[s].append(out[cu[e]:cu[e + 1]].cpu())
    for s, toks in seqs.items():
        rows = plain.bigram_rows(toks, buckets, mp, mc)
        ref = table.double()[toks] + pair.double()[rows]
        close(torch.cat(got[s]), ref, torch.float32, what="pair embedding, slot %d" % s)
    assert last.tolist() == [seqs[0][-1], -7, seqs[2][-1]]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,H", [(13, 50), (5, 2048), (70, 1100), (200, 4096), (3, 5000)])
def test_stream_kernels(dtype, T, H):
    """Rows whose values a thread keeps in registers, rows shared by several blocks (few rows), and the plain loop."""
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(2)
    eps = 1e-5
    base, y = torch.randn((T, H), generator=g), (3 * torch.randn((T, H), generator=g)).to(DT[dtype])
    w = (1 + 0.2 * torch.randn((H,), generator=g)).to(DT[dtype])
    out, copy = ops.norm_residual(base.to(dev), y.to(dev), w.to(dev), eps, None, DT[dtype])
    ref = base.double() + plain.rms_norm(y.double(), w.double(), eps)
    close(out, ref, torch.float32, what="norm_residual")
    if copy is not None:
        close(copy, ref, torch.bfloat16, what="norm_residual copy")
    kept = torch.randn((6, T, H), generator=g)
    a = torch.randn((4,), generator=g).to(DT[dtype])
    # the same sum formed by the kernel that writes the newest of the kept results
    held = kept.clone().to(dev)
    mixed, copy = ops.norm_residual(base.to(dev), y.to(dev), w.to(dev), eps, held[3], DT[dtype], (held, 4, a.to(dev)))
    close(held[3], ref, torch.float32, what="norm_residual into a kept result")
    want = sum(a[j].double() * kept[j].double() for j in range(3)) + a[3].double() * ref
    close(mixed, want, torch.float32, what="norm_residual with the mix")
    if copy is not None:
        close(copy, want, torch.bfloat16, what="copy of the mix")
    out, _ = ops.depth_mix(kept.to(dev), 4, a.to(dev), DT[dtype])
    close(out, sum(a[j].double() * kept[j].double() for j in range(4)), torch.float32, what="depth_mix")
    z = (2 * torch.randn((T, H), generator=g)).to(DT[dtype])
    for pq in ((0.3, -0.4), (-2.0, 1.5)):
        t = torch.tensor(pq).to(DT[dtype])
        got = ops.xielu(z.clone().to(dev), t.to(dev))
        close(got, plain.xielu(z.double(), float(t[0]), float(t[1])), DT[dtype], what="xielu %r" % (pq,))


@pytest.mark.parametrize("W", [70, 33, 512])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mingru_scan_in_pieces_carries_the_state(dtype, W):
    from spyinfer_amd.engine.batch import StepBatch  # noqa: F401  (the pieces are planned as the part plans them)
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.parts import recurrent
    dev = require_gpu()
    g = torch.Generator().manual_seed(3)
    lens = [150, 1, 33]
    zxg = torch.randn((sum(lens) * 2, 3 * W), generator=g).to(DT[dtype])
    bz, bx = torch.randn((W,), generator=g).to(DT[dtype]), torch.randn((W,), generator=g).to(DT[dtype])
    state = torch.zeros((5, W), dtype=torch.float32, device=dev)
    slots = [3, 0, 4]

    class FakeBatch:
        def __init__(self, ls):
            import numpy as np
            self.S, self.lens, self.shared, self.arrays = len(ls), np.asarray(ls, dtype=np.int32), {}, {}
            self._cu = np.concatenate([[0], np.cumsum(ls)]).astype(np.int32)

        def host_array(self, name):
            return self._cu

        def add_array(self, name, values):
            self.arrays[name] = values
    outs, row = [[] for _ in lens], 0
    for step in range(2):                                   # two steps: the second starts from the first's state
        fb = FakeBatch(lens)
        recurrent.plan_scan_pieces(fb)
        n, multi = fb.shared["scan_pieces"]
        assert multi and n == sum(-(-l // recurrent.SCAN_PIECE) for l in lens)
        x = zxg[row:row + sum(lens)]
        y = ops.mingru(x.to(dev), bz.to(dev), bx.to(dev), state, i32(fb.arrays["scan_pieces"], dev), n, multi, i32(slots, dev))
        at = 0
        for e, l in enumerate(lens):
            outs[e].append((x[at:at + l], y[at:at + l].cpu()))
            at += l
        row += sum(lens)
    for e in range(len(lens)):
        x = torch.cat([a for a, _ in outs[e]]).double()
        z = torch.sigmoid(x[:, :W] + bz.double())
        u = x[:, W:2 * W] + bx.double()
        c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
        s, ref = torch.zeros(W, dtype=torch.float64), []
        for t in range(x.shape[0]):
            s = (1 - z[t]) * s + z[t] * c[t]
            ref.append(s * x[t, 2 * W:] * torch.sigmoid(x[t, 2 * W:]))
        close(torch.cat([b for _, b in outs[e]]), torch.stack(ref), DT[dtype], what="mingru entry %d" % e)
        close(state[slots[e]], s, torch.float32, what="mingru state %d" % e)


@pytest.mark.parametrize("case", [dict(H=16, R=512, DR=64, P=16, window=300, entries=[(700, 1), (40, 1), (299, 1), (1500, 1)], parts=6),
                                  dict(H=16, R=512, DR=64, P=16, window=300, entries=[(0, 350), (811, 5), (64, 1)], parts=1),
                                  dict(H=5, R=96, DR=32, P=8, window=None, entries=[(0, 70), (130, 3), (257, 1)], parts=3),
                                  dict(H=72, R=40, DR=8, P=32, window=33, entries=[(100, 1), (0, 45)], parts=2),
                                  dict(H=16, R=512, DR=64, P=16, window=200, entries=[(0, 300), (500, 37), (64, 1)], parts=1, tile=128),
                                  dict(H=6, R=64, DR=16, P=8, window=None, entries=[(0, 90), (130, 3)], parts=2, tile=128)])
def test_latent_attention_on_mfma_equals_the_plain_kernel(case):
    """Rows of real sizes, a sink, a window that begins and ends inside pages and chunks, entries that are single tokens
    far into a request or portions from its start, keys in parts: against the float32 kernel on the same cache."""
    import numpy as np
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(5)
    H, R, DR, P, window = case["H"], case["R"], case["DR"], case["P"], case["window"]
    D = R + DR
    S = len(case["entries"])
    lens = [n for _, n in case["entries"]]
    kv = [p0 + n for p0, n in case["entries"]]
    T = sum(lens)
    width = max(-(-k // P) for k in kv)
    pages = sum(-(-k // P) for k in kv) + 3
    perm = torch.randperm(pages, generator=g).tolist()
    table = np.full((S, width), -1, dtype=np.int32)
    for s, k in enumerate(kv):
        for b in range(-(-k // P)):
            table[s, b] = perm.pop()
    cache = torch.randn((pages, P, D), generator=g).to(torch.bfloat16).to(dev)
    qa = (3.0 * torch.randn((T, H, D), generator=g) / D ** 0.5).to(dev)
    sink = torch.randn((H,), generator=g).to(torch.bfloat16).to(dev)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    ent = np.repeat(np.arange(S, dtype=np.int32), lens)
    pos = np.concatenate([np.arange(p0, p0 + n) for p0, n in case["entries"]]).astype(np.int32)
    meta = ops.AttentionMeta(i32(cu, dev), i32([p0 for p0, _ in case["entries"]], dev), i32(kv, dev), torch.tensor(table, device=dev),
                             i32(ent, dev), i32(pos, dev), S, T, width, max(kv), max(lens))
    size = case.get("tile", ops.LATENT_TILE_ROWS)
    counts = [-(-n * H // size) for n in lens]
    tiles = (i32(np.repeat(np.arange(S), counts), dev), i32(np.concatenate([np.arange(c) * size for c in counts]), dev), sum(counts), size)
    ref = ops.latent_attention(qa, cache, P, meta, sink, R, 0.7, window, torch.float32)
    got = ops.latent_attention(qa.to(torch.bfloat16), cache, P, meta, sink, R, 0.7, window, torch.bfloat16, tiles, case["parts"])
    close(got, ref, torch.bfloat16, what="latent attention on MFMA")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("dims,scaling", [(8, None), (6, dict(factor=8.0, original=64, fast=16.0, slow=2.0)), (0, None)])
def test_latent_prepare_norms_rotates_and_stores(dtype, dims, scaling):
    """The latent's norm, the rotation (all of the rotated part or its first dims, with and without scaled frequencies,
    or none) of the shared key part and of every head's query part, and the store into the tokens' page rows."""
    from spyinfer_amd.kernels import ops
    from spyinfer_amd.parts import RotaryEmbedding
    dev = require_gpu()
    g = torch.Generator().manual_seed(7)
    T, H, DN, DR, R, P, eps = 11, 3, 6, 8, 20, 4, 1e-5
    ld = H * (DN + DR) + R + DR
    qd = torch.randn((T, ld), generator=g).to(DT[dtype])
    w = (1 + 0.3 * torch.randn((R,), generator=g)).to(DT[dtype])
    pos = torch.tensor([0, 1, 2, 3, 4, 700, 701, 702, 9000, 9001, 33], dtype=torch.int32)
    slots = torch.randperm(6 * P, generator=g)[:T].to(torch.int32)
    cache = torch.full((6, P, R + DR), float("nan"), dtype=DT[dtype], device=dev)
    freq = mag = None
    if dims:
        rot = RotaryEmbedding(DR, 5000.0, dims, scaling)
        rot.prepare(dev, 0)
        freq, mag, _ = rot.frequencies()
    x = qd.to(dev)
    qa = ops.latent_prepare(x, x[:, H * (DN + DR):], cache, slots.to(dev), w.to(dev), eps, freq, mag or 1.0, dims, pos.to(dev), H, DN, DR, R,
                            DT[dtype])
    d = qd.double()[:, H * (DN + DR):]
    c_ref = plain.rms_norm(d[:, :R], w.double(), eps)
    q_rot = qd.double()[:, :H * (DN + DR)].view(T, H, DN + DR)[:, :, DN:]
    kr_ref = d[:, R:]
    if dims:
        f, m = plain.yarn_frequencies(dims, 5000.0, scaling)
        kr_ref = plain.rotate_half(kr_ref, pos, f, m, dims)
        q_rot = plain.rotate_half(q_rot.transpose(0, 1), pos, f, m, dims).transpose(0, 1)
    rows = cache.view(-1, R + DR)[slots.long().to(dev)]
    # angles are position * frequency in float32: at position 9000 that alone is 1e-3 of a turn's sine
    tol = torch.float32 if dtype == "float32" else torch.bfloat16
    close(rows[:, :R], c_ref, tol, what="latent")
    close(rows[:, R:], kr_ref, tol, scale=40.0 if dtype == "float32" else 1.0, what="rotated key part")
    close(qa[:, :, R:], q_rot, tol, scale=40.0 if dtype == "float32" else 1.0, what="rotated query parts")
    untouched = torch.ones(6 * P, dtype=torch.bool)
    untouched[slots.long()] = False
    assert torch.isnan(cache.view(-1, R + DR)[untouched.to(dev)]).all(), "a row of another token was written"


@pytest.mark.parametrize("T,H,N,K,out_dtype", [(1, 16, 512, 128, torch.bfloat16), (37, 3, 40, 72, torch.float32), (128, 8, 128, 512, torch.bfloat16)])
def test_head_products(T, H, N, K, out_dtype):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(6)
    pad = 24                                              # the rows of x are views into wider rows
    x = torch.randn((T, H * (K + pad)), generator=g).to(torch.bfloat16).to(dev)
    w = (torch.randn((H, N, K), generator=g) / K ** 0.5).to(torch.bfloat16).to(dev)
    out = torch.zeros((T, H, N + 4), dtype=out_dtype, device=dev)
    ops.head_products(x, H * (K + pad), K + pad, w, out, H * (N + 4), N + 4, T)
    ref = torch.einsum("thk,hnk->thn", x.view(T, H, K + pad)[:, :, :K].double().cpu(), w.double().cpu())
    close(out[:, :, :N], ref, out_dtype if out_dtype == torch.bfloat16 else torch.float32, what="head_products")
    assert float(out[:, :, N:].abs().max()) == 0.0


@pytest.mark.parametrize("M", [1, 8, 16, 17, 40, 64])
@pytest.mark.parametrize("N,K", [(256, 256), (3072, 1024), (6144, 512)])
def test_decode_product_with_the_activation_in_its_epilogue(M, N, K):
    from spyinfer_amd.kernels import ops
    dev = require_gpu()
    g = torch.Generator().manual_seed(8)
    x = torch.randn((M, K), generator=g).to(torch.bfloat16)
    w = (torch.randn((N, K), generator=g) / K ** 0.5).to(torch.bfloat16)
    pq = torch.tensor([0.4, -0.7]).to(torch.bfloat16)
    tiled = ops.tile_weight(w.to(dev))
    assert tiled is not None
    got = ops.linear_xielu(x.to(dev), w.to(dev), pq.to(dev), tiled)
    ref = plain.xielu(x.double() @ w.double().T, float(pq[0]), float(pq[1]))
    close(got, ref, torch.bfloat16, what="up product with xIELU, %d rows" % M)
    # and the same through the separate kernel
    close(ops.xielu(ops.linear_few(x.to(dev), w.to(dev), tiled), pq.to(dev)), ref, torch.bfloat16, what="product, then xIELU")


# ---- whole models under every schedule ------------------------------------------------------------
MODELS = {"a": (sc.SEF_A, 3, None), "b": (sc.SEF_B, 4, None), "c": (sc.SEF_C, 6, None), "a_sharp": (sc.SEF_A, 5, sc.sharpen()),
          "c_sink": (sc.SEF_C, 9, sc.heavy_sinks()), "long_sharp": (sc.SEF_LONG, 10, sc.sharpen(4.0)),
          "far_sharp": (sc.SEF_FAR, 8, sc.sharpen(8.0))}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: sc.write_model(str(tmp_path_factory.mktemp("gsef_" + name)), cfg, seed, tweak) for name, (cfg, seed, tweak) in MODELS.items()}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["a", "b", "c", "a_sharp", "c_sink"])
@pytest.mark.parametrize("mode", ["whole", "bulk_tail", "portions", "mixed"])
def test_schedules_equal_the_plain_implementation(folders, name, mode, dtype, tmp_path):
    require_gpu()
    folder = folders[name]
    requests = rc.random_requests(sc.vocab_of(folder), [41, 1, 2, 130, 23, 30, 52, 38, 75], 7)
    steps = {"whole": rc.whole, "bulk_tail": lambda r: rc.bulk_tail(r, 40), "portions": rc.portions, "mixed": rc.mixed}[mode](requests)
    rc.run_replay_inprocess(folder, dtype, str(tmp_path), steps, rc.max_live_tokens(steps),
                            ["--kvcache-block-size", "8" if not name.startswith("c") else "16", "--poison-cache"])
    rc.compare(rc.collect(str(tmp_path), steps, sc.vocab_of(folder)), sc.plain_logits(folder, requests),
               what="%s/%s/%s" % (name, mode, dtype), **TOL[dtype])


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
    """Requests of up to 1200 tokens, windows of 333 and 150 tokens on the same rows, sharp scores; decoding passes the
    windows' edges over prompt tokens and decoded ones; four such requests share pages and slots in the mixed schedule."""
    require_gpu()
    folder = folders["long_sharp"]
    requests = rc.random_requests(211, [1200, 400, 700, 3, 520], 21)
    steps = {"whole": rc.whole, "bulk_tail": lambda r: rc.bulk_tail(r, 200), "portions": lambda r: rc.portions(r, (300, 2, 129, 64, 5, 411, 33)),
             "mixed": lambda r: rc.mixed(r, seed=3)}[mode](requests)
    rc.run_replay_inprocess(folder, dtype, str(tmp_path), steps, rc.max_live_tokens(steps), ["--poison-cache"])
    tol = TOL[dtype] if dtype == "float32" else dict(atol=0.25, rtol=5e-2)
    rc.compare(rc.collect(str(tmp_path), steps, 211), sc.plain_logits(folder, requests), what="long/%s/%s" % (mode, dtype), **tol)


def test_long_decoding_passes_many_windows(folders, tmp_path):
    require_gpu()
    folder = folders["a"]
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
    model = plain.PlainSefevik.from_folder(folder)
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
    model = plain.PlainSefevik.from_folder(folder)
    prompts = list(rc.random_requests(400, [33, 70, 8], 10).values())
    eng = LLMEngine(folder, dtype="bfloat16", max_model_len=128, num_kvcache_blocks=40, max_num_seqs=4)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=12, ignore_eos=True))
    for p, out in zip(prompts, outs):
        toks = list(p)
        for t in out:
            logits = model.forward(toks)[-1]
            best = int(torch.argmax(logits))
            assert t == best or float(logits[best] - logits[t]) < 0.15, "token %d where the plain logits prefer %d clearly" % (t, best)
            toks.append(t)


def test_trace_run_as_a_program(folders, tmp_path):
    require_gpu()
    folder = folders["b"]
    requests = rc.random_requests(61, [19, 40], 14)
    steps = rc.portions(requests)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    import json
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
