"""Kuponex on the GPU against the plain float64 implementation (plain_kuponex): every mechanism alone, whole
prompts against token-by-token decoding and against portions of several sizes, batches of unequal requests
against each alone with pages and slots that are used again, far keys and the sink made to matter, long
decoding, and greedy generation through the engine."""

import json
from pathlib import Path

import numpy as np
import pytest
import torch

import bitwise_amd as bw
import plain_kuponex as pk

pytestmark = pytest.mark.gpu

# float32: a row now and then sits where a head's read-out nearly cancels and the 32-bit sums' last bits show (a few 1e-5); the
# bulk is held to 5e-6.
# bfloat16: against the plain model rounded at the engine's rounding points; what is left are the queries and softmax
# weights that the matrix-core attention rounds on their way into its products, and roundings that fall the other way
# because 32-bit sums differ from exact ones in their last bits (some 5e-3 a row in a model of several layers, a few
# 1e-2 in a row now and then; a mechanism that is wrong moves a row by its own size and shows in 32-bit first)
TOL = {"float32": 1e-4, "bfloat16": 5e-2}
TYPICAL = {"float32": 5e-6, "bfloat16": 1e-2}
RND = {"float32": pk.identity, "bfloat16": pk.round_bf16}
SIGMA = 0.15


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base, dims, ff):
    return {"type": "latent_attention", "mlp": None if ff is None else {"kind": "dense", "ff": ff},
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                      "rot": {"base": base, "dims": dims}}}


def gla(heads, dim, vdim, tau, rank, ff):
    return {"type": "gla", "mlp": None if ff is None else {"kind": "dense", "ff": ff},
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "rank": rank}}


def mlstm(heads, dim, vdim, cap, ff):
    return {"type": "mlstm", "mlp": None if ff is None else {"kind": "dense", "ff": ff},
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}}


def config(width, vocab, eps, layers):
    return {"architecture": "Kuponex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers, "max_positions": 2048}


CONFIGS = {
    # one mixer each, no feed-forward: the mechanism alone
    "only_gla": config(48, 61, 1e-5, [gla(3, 8, 20, 4.0, 5, None)]),
    "only_mlstm": config(48, 61, 1e-5, [mlstm(3, 8, 20, 6.0, None)]),
    "only_latent": config(48, 61, 1e-5, [latent(3, 8, 8, 12, 24, 0.3, 300.0, 8, None)]),
    "only_latent_odd": config(48, 61, 1e-5, [latent(5, 6, 6, 10, 21, 0.3, 300.0, 6, None)]),      # a key vector that is no multiple of 8
    # more heads than a wave's 16 query vectors (a second, partly filled group), tiny heads; eps that matters
    "many_heads": config(40, 67, 1e-2, [latent(18, 4, 4, 4, 12, 0.5, 50.0, 4, 48), gla(5, 8, 4, 2.0, 2, None), mlstm(6, 4, 12, 3.0, 32)]),
    # everything together, sizes all different, a partly rotated key part, a layer without feed-forward, one head
    "mixed": config(64, 131, 1e-5, [mlstm(2, 16, 24, 8.0, 96), latent(3, 8, 8, 20, 24, 0.2, 500.0, 4, 80),
                                     gla(4, 8, 8, 4.0, 3, None), latent(1, 16, 4, 8, 12, 0.25, 10000.0, 4, 72),
                                     gla(1, 24, 40, 32.0, 8, 56)]),
    # sizes beyond a wave: value columns in two blocks, key channels over two registers a lane, heads that fill no group
    "wide": config(96, 77, 1e-6, [gla(2, 40, 72, 8.0, 6, 120), mlstm(2, 72, 40, 12.0, 64),
                                   latent(5, 12, 16, 24, 72, 0.15, 2000.0, 16, 104), mlstm(1, 8, 136, 20.0, None)]),
}
SEEDS = {"only_gla": 11, "only_mlstm": 12, "only_latent": 13, "only_latent_odd": 14, "mixed": 15, "wide": 16, "many_heads": 17}


@pytest.fixture(scope="module")
def folders(tmp_path_factory, gpu):
    tmp = tmp_path_factory.mktemp("kuponex")
    return {name: bw.write_random_model(tmp / name, cfg, SEEDS[name], SIGMA) for name, cfg in CONFIGS.items()}


def weights(folder):
    from safetensors.torch import load_file
    return pk.to64(load_file(str(Path(folder) / "model.safetensors")))


def tokens_for(name, n, seed=0):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, CONFIGS[name]["vocab"], (n,), generator=g).tolist()


def plain(name, folder, toks, dtype="float32"):
    return pk.forward(json.loads((Path(folder) / "config.json").read_text()), weights(folder), toks, rnd=RND[dtype]).numpy()


def close(got, want, dtype):
    worst = pk.logits_error(got, want)
    typical = pk.logits_error(got, want, quantile=0.5)
    return worst < TOL[dtype] and typical < TYPICAL[dtype]


def replayer(folder, dtype, max_tokens, **kw):
    from bitwise_amd.replay import Replayer
    return Replayer(str(folder), dtype, max_tokens, max_live=4, **kw)


def run_cut(rp, rid, toks, cuts):
    """One request through a replayer in portions of the given sizes (the rest one by one); logits at every position."""
    out, at = [], 0
    sizes = list(cuts) + [1] * (len(toks) - sum(cuts))
    for n in sizes:
        out.append(rp.step([{"id": rid, "tokens": toks[at:at + n], "want": list(range(n))}]))
        at += n
    rp.step([], [rid])
    return np.concatenate(out)


# ----------------------------------------------------------------------------- the model against the plain one

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompts_equal_plain(folders, name, dtype):
    model = bw.Model.load(folders[name], dtype)
    for n, seed in ((1, 0), (2, 1), (37, 2), (150, 3)):
        toks = tokens_for(name, n, seed)
        got = model.logits(toks)
        assert close(got, plain(name, folders[name], toks, dtype), dtype), (name, n)
    assert model.weight_bytes > 0 and model.config.width == CONFIGS[name]["width"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "wide"])
def test_decoding_and_portions_equal_the_whole_prompt(folders, name, dtype):
    """Token by token from the first token on, a prompt then single tokens, and portions down to two tokens whose
    edges fall inside pages: the logits of every position stay those of the whole prompt, with graphs and without."""
    toks = tokens_for(name, 83, 5)
    want = plain(name, folders[name], toks, dtype)
    cuttings = ([], [83], [51], [2, 2, 3, 16, 17, 2, 30, 5], [15, 1, 1, 33, 2], [64, 2])
    for graphs in (True, False):
        rp = replayer(folders[name], dtype, 256, use_graphs=graphs, poison_freed_pages=True)
        for k, cuts in enumerate(cuttings):
            got = run_cut(rp, f"r{k}", toks, cuts)
            assert close(got, want, dtype), (name, graphs, cuts)
        assert rp.manager.all_free()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_requests_together_equal_each_alone(folders, dtype):
    """Four live requests of different lengths, portions beside single tokens, requests that pause, end and are followed
    by others in the same slots and pages (freed pages are filled with NaN at once): every position as alone."""
    name = "mixed"
    lengths = {"a": 70, "b": 9, "c": 33, "d": 1, "e": 48, "f": 21}
    toks = {r: tokens_for(name, n, 20 + i) for i, (r, n) in enumerate(lengths.items())}
    want = {r: plain(name, folders[name], t, dtype) for r, t in toks.items()}
    rp = replayer(folders[name], dtype, 64 * 4, poison_freed_pages=True)
    plan = [  # (request, tokens) per step
        [("a", 17), ("b", 2), ("c", 5), ("d", 1)],
        [("a", 1), ("b", 1), ("c", 16)],
        [("a", 30), ("b", 6), ("e", 2)],             # d has ended: e takes its slot; c pauses
        [("a", 1), ("c", 12), ("e", 31), ("f", 3)],  # b has ended
        [("a", 21), ("e", 1), ("f", 18)],
        [("e", 14)],
    ]
    at = {r: 0 for r in toks}
    got = {r: [] for r in toks}
    slots_used = {}
    for step in plan:
        entries, ends = [], []
        for r, n in step:
            entries.append({"id": r, "tokens": toks[r][at[r]:at[r] + n], "want": list(range(n))})
            at[r] += n
            if at[r] == lengths[r]:
                ends.append(r)
        lg = rp.step(entries, [])
        for r in (e["id"] for e in entries):
            slots_used[r] = rp.live[r].slot
        row = 0
        for r, n in step:
            got[r].append(lg[row:row + n])
            row += n
        rp.step([], ends)
    assert at == lengths and rp.manager.all_free()
    assert len(set(slots_used.values())) < len(slots_used), "slots were meant to be used again"
    for r in toks:
        assert close(np.concatenate(got[r]), want[r], dtype), r


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """300 tokens one by one behind a short prompt, across many pages and blocks of keys: no drift in the states."""
    name = "wide"
    toks = tokens_for(name, 330, 7)
    rp = replayer(folders[name], dtype, 384)
    got = run_cut(rp, "x", toks, [30])
    assert close(got, plain(name, folders[name], toks, dtype), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_portions_beside_short_ones(folders, dtype):
    """Portions long enough for the recurrences' three passes over chunks (whole, cut at and beside a chunk's edge), alone and
    in one step with a short portion and a single token of other requests; the engine that runs them allows logits to depend
    on the cut in their last bits (``exact_cuts=False``).  With the default the cuttings agree bit for bit."""
    name = "wide"
    toks = tokens_for(name, 330, 31)
    want = plain(name, folders[name], toks, dtype)
    rp = replayer(folders[name], dtype, 1024, exact_cuts=False)
    for k, cuts in enumerate(([330], [129, 201], [128, 128, 74], [191, 130])):
        assert close(run_cut(rp, f"w{k}", toks, cuts), want, dtype), cuts
    small, one = tokens_for(name, 9, 32), tokens_for(name, 3, 33)
    rp.step([{"id": "one", "tokens": one[:2], "want": []}])
    lg = rp.step([{"id": "small", "tokens": small[:5], "want": [4]}, {"id": "long", "tokens": toks[:260], "want": [0, 127, 128, 259]},
                  {"id": "one", "tokens": one[2:], "want": [0]}])
    assert close(lg[1:5], want[[0, 127, 128, 259]], dtype)
    assert close(lg[:1], plain(name, folders[name], small, dtype)[4:5], dtype)
    assert close(lg[5:], plain(name, folders[name], one, dtype)[2:], dtype)
    lg = rp.step([{"id": "long", "tokens": toks[260:], "want": [0, 69]}, {"id": "small", "tokens": small[5:], "want": [3]}], ["long", "small", "one"])
    assert close(lg[:2], want[[260, 329]], dtype) and close(lg[2:], plain(name, folders[name], small, dtype)[8:], dtype)
    assert rp.manager.all_free()
    exact = replayer(folders[name], dtype, 1024)
    runs = [run_cut(exact, f"e{k}", toks, cuts) for k, cuts in enumerate(([330], [129, 201], [17, 300], [2] * 20))]
    assert all(np.array_equal(runs[0], r) for r in runs[1:])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(folders, dtype):
    """bw.generate with the engine's scheduler, a small token budget and a small page pool: the tokens of the plain
    implementation, which recomputes the whole sequence for every token."""
    name = "mixed"
    cfg, w = CONFIGS[name], weights(folders[name])
    model = bw.Model.load(folders[name], dtype)
    prompts = [tokens_for(name, n, 40 + n) for n in (1, 6, 19, 40)]
    sp = bw.SamplingParams(max_new_tokens=12, ignore_eos=True)
    results = bw.generate(model, prompts, sp, bw.EngineConfig(num_blocks=16, max_batched_tokens=24, max_num_seqs=3, dtype=dtype))
    for p, r in zip(prompts, results):
        assert r.finished and len(r.tokens) == 12
        if dtype == "float32":
            assert r.tokens == pk.generate_greedy(cfg, w, p, 12)
    # the same requests alone, graphs off: the same tokens and logits to the last bit
    for p, r in zip(prompts, results):
        solo = bw.generate(model, [p], sp, bw.EngineConfig(num_blocks=16, max_num_seqs=1, dtype=dtype, use_graphs=False))[0]
        assert solo.tokens == r.tokens and solo.logits_fingerprint == r.logits_fingerprint


def test_engine_preemption_recomputes_state(folders):
    """A page pool too small for all requests: a preempted request gives its slot back, starts again from zeroed state
    and ends with the tokens of a run alone."""
    name, dtype = "mixed", "float32"
    model = bw.Model.load(folders[name], dtype)
    prompts = [tokens_for(name, n, 60 + n) for n in (9, 17, 5, 12)]
    sp = bw.SamplingParams(max_new_tokens=20, ignore_eos=True)
    solo = [bw.generate(model, [p], sp, bw.EngineConfig(num_blocks=8, max_num_seqs=1, dtype=dtype))[0] for p in prompts]
    eng = bw.Engine(model, None, bw.EngineConfig(num_blocks=7, max_batched_tokens=16, max_num_seqs=4, dtype=dtype))
    ids = [eng.add_request(p, sp) for p in prompts]
    guard = 0
    while not eng.idle():
        eng.step()
        guard += 1
        assert guard < 2000
    assert eng.stats.preemptions > 0, "the pool was meant to be too small"
    for i, ref in zip(ids, solo):
        assert eng.result(i).tokens == ref.tokens and eng.result(i).logits_fingerprint == ref.logits_fingerprint
    assert eng.manager.all_free()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_randomized_scenarios_to_the_last_bit(gpu, dtype):
    """The scenario simulator on the architecture's tiny model: page sizes, graphs, pools and budgets drawn per scenario,
    every request against its solo run: no wrong token, no other logits (the default engine promises bits under any cut),
    no page or slot lost; preemption happens on the way and restarts from zeroed state."""
    from bitwise_amd.registry import ARCHITECTURES
    from bitwise_amd.sim import Simulator

    model = bw.Model.random(ARCHITECTURES["Kuponex"].tiny_config, 42, dtype, sigma=0.08)
    tally = Simulator(model, dtype).run(16, seed=1)
    print(tally.line(dtype))
    assert tally.violations() == 0, "\n".join(tally.notes[:10])
    assert tally.requests_compared > 40 and tally.preemptions > 0 and tally.prefix_hit_tokens == 0


# ----------------------------------------------------------------------------- mechanisms made to matter

def _attend(q, keys, sink, heads, dk, dv, scale, page, dtype, positions, window=0, matrix_cores=None):
    """shared_key_attention for single rows of one request at the given positions over ``keys`` [n, dk].  ``matrix_cores``:
    (heads per group, splits) runs the matrix-core kernel instead."""
    from bitwise_amd.csrc import ops
    dev = torch.device("cuda:0")
    n = keys.shape[0]
    pages = (n + page - 1) // page
    order = torch.randperm(pages, generator=torch.Generator().manual_seed(3))     # the request's pages lie scattered
    cache = torch.zeros(pages, page * dk, dtype=dtype)
    padded = torch.zeros(pages * page, dk, dtype=torch.float64)
    padded[:n] = keys
    for i in range(pages):
        cache[order[i]] = padded[i * page:(i + 1) * page].reshape(-1).to(dtype)
    table = order.to(torch.int32).view(1, -1).to(dev)
    rows = len(positions)
    out = torch.zeros(rows, heads * dv, device=dev)
    pos = torch.tensor(positions, dtype=torch.int32, device=dev)
    tiles = torch.tensor([[r, 1, 0, 0] for r in range(rows)], dtype=torch.int32, device=dev)
    sk = None if sink is None else sink.float().to(dev)
    if matrix_cores is None:
        ops.shared_key_attention(q.float().to(dev).contiguous(), pos, table, tiles, rows, cache.to(dev), sk,
                                 out, heads, dk, dv, page, window, scale, 16)
    else:
        hg, nsplit = matrix_cores
        vt = cache.view(pages, page, dk)[:, :, :dv].transpose(1, 2).contiguous().view(pages, dv * page)
        kchunk = 64 * max(1, -(-(pages * page) // (64 * nsplit)))
        nsplit = -(-(pages * page) // kchunk)
        partial = torch.zeros(rows * heads * nsplit * (dv + 2), device=dev) if nsplit > 1 else None
        ops.shared_key_attention_mfma(q.bfloat16().to(dev).contiguous(), pos, table, tiles, rows, cache.to(dev), vt.to(dev), sk, out,
                                      heads, dk, dv, page, window, scale, hg, nsplit, kchunk, partial)
    return out.cpu().double().view(rows, heads, dv), cache


def _attend_plain(q, keys, sink, heads, dk, dv, scale, positions, window=0):
    out = torch.zeros(len(positions), heads, dv, dtype=torch.float64)
    for r, p in enumerate(positions):
        lo = max(0, p - window + 1) if window else 0
        k = keys[lo:p + 1]
        s = torch.einsum("hd,jd->hj", q[r].view(heads, dk), k) * scale
        if sink is not None:
            s = torch.cat([s, sink.view(heads, 1)], 1)
        wgt = torch.softmax(s, -1)
        out[r] = wgt[:, :k.shape[0]] @ k[:, :dv]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds_and_page_borders(gpu, dtype):
    """One query per probe is a scaled copy of one key far back (the first key, keys just before and after a page's
    border, the one before the last), so that this key carries the weight: a key that is lost or taken from a wrong page
    slot shows."""
    g = torch.Generator().manual_seed(5)
    heads, dk, dv, page, n = 5, 40, 24, 16, 700
    keys = torch.randn(n, dk, generator=g, dtype=torch.float64)
    if dtype == torch.bfloat16:
        keys = keys.bfloat16().double()
    targets = [0, 1, 15, 16, 17, 63, 64, 65, 300, 511, 512, 640, 698, 699]
    positions = [n - 1] * len(targets)
    q = torch.randn(len(targets), heads * dk, generator=g, dtype=torch.float64) * 0.1
    for r, t in enumerate(targets):
        q[r].view(heads, dk)[r % heads] += 3.0 * keys[t]
    sink = torch.randn(heads, generator=g, dtype=torch.float64)
    got, _ = _attend(q, keys, sink, heads, dk, dv, 0.2, page, dtype, positions)
    want = _attend_plain(q.float().double(), keys, sink, heads, dk, dv, 0.2, positions)
    assert (got - want).abs().max() < 2e-5 * want.abs().max() + 1e-5
    for r, t in enumerate(targets):       # the probe's head returns (nearly) the value of its target
        assert (got[r, r % heads] - keys[t, :dv]).abs().max() < 0.05, t
    if dtype == torch.bfloat16:
        # the matrix-core kernel: whole key range by one wave, and cut into pieces that a second kernel joins; queries and
        # weights are rounded to bfloat16 on their way into the products
        qr = q.bfloat16().double()
        want = _attend_plain(qr, keys, sink, heads, dk, dv, 0.2, positions)
        for route in ((8, 1), (16, 1), (16, 4), (16, 11)):
            got, _ = _attend(q, keys, sink, heads, dk, dv, 0.2, page, dtype, positions, matrix_cores=route)
            assert (got - want).abs().max() < 1e-2 * want.abs().max(), route
            for r, t in enumerate(targets):
                assert (got[r, r % heads] - keys[t, :dv]).abs().max() < 0.05, (route, t)


def test_the_sink_takes_weight_and_a_window_cuts_keys(gpu):
    g = torch.Generator().manual_seed(6)
    heads, dk, dv, page, n = 3, 24, 24, 8, 90
    keys = torch.randn(n, dk, generator=g, dtype=torch.float64)
    positions = [0, 1, 7, 8, 40, 89]
    q = torch.randn(len(positions), heads * dk, generator=g, dtype=torch.float64)
    big = torch.tensor([9.0, 0.0, -30.0], dtype=torch.float64)
    with_sink, _ = _attend(q, keys, big, heads, dk, dv, 0.3, page, torch.float32, positions)
    without, _ = _attend(q, keys, None, heads, dk, dv, 0.3, page, torch.float32, positions)
    for sink, got in ((big, with_sink), (None, without)):
        want = _attend_plain(q.float().double(), keys, sink, heads, dk, dv, 0.3, positions)
        assert (got - want).abs().max() < 2e-5 * want.abs().max() + 1e-6
    assert with_sink[:, 0].abs().max() < 0.2 * without[:, 0].abs().max()       # a large sink leaves little for the values
    assert (with_sink[:, 2] - without[:, 2]).abs().max() < 1e-3                 # a very negative one changes nothing
    # a window: the key just inside counts, the one just outside does not
    W = 13
    keys2 = keys.clone()
    keys2[89 - W] += 50.0          # just outside the window of position 89, inside that of position 88
    got, _ = _attend(q[:2].repeat(1, 1), keys2, None, heads, dk, dv, 0.3, page, torch.float32, [89, 88], window=W)
    want = _attend_plain(q[:2].float().double(), keys2, None, heads, dk, dv, 0.3, [89, 88], window=W)
    assert (got - want).abs().max() < 2e-5 * want.abs().max() + 1e-6


def test_recurrences_remember_the_first_token(folders):
    """A model of matrix-memory mixers whose decays are pushed towards 1: the first token still moves the logits 200
    tokens later, through a prompt and through single tokens alike (a state that is dropped or zeroed shows)."""
    from safetensors.torch import load_file, save_file
    name = "wide"
    src = Path(folders[name])
    dst = src.parent / "wide_long_memory"
    dst.mkdir(exist_ok=True)
    w = load_file(str(src / "model.safetensors"))
    for k in w:
        if k.endswith("a2.b") or k.endswith("f.b"):
            w[k] = torch.full_like(w[k], 8.0)
    save_file(w, str(dst / "model.safetensors"))
    (dst / "config.json").write_text((src / "config.json").read_text())
    toks = tokens_for(name, 200, 9)
    other = [(toks[0] + 1) % CONFIGS[name]["vocab"]] + toks[1:]
    cfg, w64 = CONFIGS[name], pk.to64(w)
    want, want_other = pk.forward(cfg, w64, toks).numpy(), pk.forward(cfg, w64, other).numpy()
    assert pk.logits_error(want_other[-1:], want[-1:]) > 1e-3, "the first token was meant to matter at the end"
    rp = replayer(dst, "float32", 256)
    for cuts in ([200], [3], [64, 64, 64]):
        assert pk.logits_error(run_cut(rp, "m", toks, cuts), want) < TOL["float32"]
        assert pk.logits_error(run_cut(rp, "o", other, cuts), want_other) < TOL["float32"]
