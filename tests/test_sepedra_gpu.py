"""Sepedra on the GPU against the plain float64 implementation (plain_sepedra): every mechanism alone (kernels and
one-layer models), whole prompts against token-by-token decoding and against portions down to two tokens, batches of
unequal requests against each alone with pages and slots that are used again, far keys, page borders and the sink made
to matter, long decoding, a recurrence that remembers its first token, and greedy generation through the engine."""

import json
from pathlib import Path

import numpy as np
import pytest
import torch

import bitwise_amd as bw
import plain_sepedra as ps

pytestmark = pytest.mark.gpu

# float32: 32-bit sums against float64 ones, a few 1e-6 of a row (observed: 9e-6 at worst); every row is held to 1e-4, so a
# mechanism that is wrong shows here first.  bfloat16: against the plain model rounded at the engine's rounding points.
# Every sublayer's output is normed to unit size on its way into the stream, so a rounding that falls the other way
# is carried at its relative size through every later layer (observed medians: 5e-3 to 2e-2 of a row), and a row whose
# router scores nearly tie picks another expert in one of the two and moves by its own size (about one row in a hundred
# where a row has one expert): the median over the rows and their 90th percentile are held, not the worst row.
TOL = {"float32": 1e-4, "bfloat16": 0.12}
WORST_QUANTILE = {"float32": 1.0, "bfloat16": 0.9}
TYPICAL = {"float32": 1e-5, "bfloat16": 3e-2}
RND = {"float32": ps.identity, "bfloat16": ps.round_bf16}
SIGMA = 0.15


def rot(base, dims, scaling=None):
    out = {"base": base, "dims": dims}
    if scaling:
        out["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return out


def attn(heads, kv_heads, dim, vdim, conv, scale, rotary, mlp=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale, "rot": rotary}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def rglru(inner, blocks, conv, mlp=None):
    return {"type": "rglru", "mixer": {"width": inner, "blocks": blocks, "conv": conv}, "mlp": mlp}


def moe(experts, top, ff, limit, groups=None):
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": router}


def config(width, vocab, eps, cap, layers):
    return {"architecture": "Sepedra", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_softcap": cap, "layers": layers,
            "max_positions": 2048}


R1 = rot(300.0, 8, (3.0, 1.0, 3.0, 40))
R2 = rot(10000.0, 12)
R3 = rot(500.0, 32, (8.0, 0.5, 6.0, 128))
CONFIGS = {
    # one mechanism each
    "only_rglru": config(48, 61, 1e-5, 15.0, [rglru(40, 5, 4)]),
    "only_attention": config(48, 61, 1e-5, 15.0, [attn(4, 2, 16, 16, 3, 0.35, R1)]),
    # (experts whose inner size is no multiple of 8: their products stay on the 32-bit kernels in bfloat16 mode too)
    "only_moe": config(48, 61, 1e-5, 15.0, [rglru(16, 1, 1, moe(8, 3, 20, 0.7, (4, 2)))]),
    # everything together, sizes all different: values wider and narrower than keys, one key head and as many as query
    # heads, a fully rotated head and a barely rotated one, no stretching, one block, one tap and five, one expert a row,
    # no groups, a layer that reads another's cache behind a recurrent layer, layers without feed-forward
    "mixed": config(64, 131, 1e-6, 25.0, [
        attn(6, 2, 12, 20, 2, 0.3, R2, moe(6, 1, 40, 1.0)),
        rglru(56, 7, 5, None),
        attn(3, 1, 24, 8, 4, 0.2, R1, moe(9, 4, 16, 3.0, (3, 2))),
        attn(6, 2, 12, 20, 3, 0.5, R2, None, kv_from=0),
        rglru(32, 1, 2, moe(4, 4, 24, 0.5, (2, 2))),
        attn(3, 1, 24, 8, 1, 0.1, R1, moe(5, 2, 8, 2.0), kv_from=2),
    ]),
    # heads of the sizes real models have, more experts than a wave has lanes, inner sizes beyond one step of the products
    "wide": config(136, 77, 1e-5, 40.0, [
        rglru(192, 3, 4, moe(72, 6, 48, 1.0, (8, 3))),
        attn(4, 4, 128, 128, 3, 0.09, rot(40000.0, 64, (6.0, 1.0, 5.0, 256)), moe(12, 3, 72, 1.5, (4, 2))),
        attn(8, 2, 64, 48, 4, 0.12, R3, None),
        attn(4, 4, 128, 128, 2, 0.05, rot(40000.0, 64, (6.0, 1.0, 5.0, 256)), moe(3, 2, 136, 4.0), kv_from=1),
    ]),
}
SEEDS = {name: 31 + i for i, name in enumerate(CONFIGS)}


@pytest.fixture(scope="module")
def folders(tmp_path_factory, gpu):
    tmp = tmp_path_factory.mktemp("sepedra")
    return {name: bw.write_random_model(tmp / name, cfg, SEEDS[name], SIGMA) for name, cfg in CONFIGS.items()}


def weights(folder):
    from safetensors.torch import load_file
    return ps.to64(load_file(str(Path(folder) / "model.safetensors")))


def tokens_for(name, n, seed=0):
    g = torch.Generator().manual_seed(2000 + seed)
    return torch.randint(0, CONFIGS[name]["vocab"], (n,), generator=g).tolist()


def plain(name, folder, toks, dtype="float32"):
    return ps.forward(json.loads((Path(folder) / "config.json").read_text()), weights(folder), toks, rnd=RND[dtype]).numpy()


def close(got, want, dtype):
    return ps.logits_error(got, want, quantile=WORST_QUANTILE[dtype]) < TOL[dtype] and ps.logits_error(got, want, quantile=0.5) < TYPICAL[dtype]


def replayer(folder, dtype, max_tokens, **kw):
    from bitwise_amd.replay import Replayer
    return Replayer(str(folder), dtype, max_tokens, max_live=4, **kw)


def run_cut(rp, rid, toks, cuts):
    """One request through a replayer in portions of the given sizes (the rest one by one); logits at every position."""
    out, at = [], 0
    for n in list(cuts) + [1] * (len(toks) - sum(cuts)):
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
        assert close(model.logits(toks), plain(name, folders[name], toks, dtype), dtype), (name, n)
    assert model.weight_bytes > 0 and model.config.width == CONFIGS[name]["width"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "wide"])
def test_decoding_and_portions_equal_the_whole_prompt(folders, name, dtype):
    """Token by token from the first token on, a prompt then single tokens, and portions down to two tokens whose edges
    fall inside pages and inside the convolutions' reach: the logits of every position stay those of the whole prompt,
    to the last bit, with graphs and without."""
    toks = tokens_for(name, 83, 5)
    want = plain(name, folders[name], toks, dtype)
    cuttings = ([83], [], [51], [2, 2, 3, 16, 17, 2, 30, 5], [15, 1, 1, 33, 2], [64, 2])
    first = None
    for graphs in (True, False):
        rp = replayer(folders[name], dtype, 256, use_graphs=graphs, poison_freed_pages=True)
        for k, cuts in enumerate(cuttings):
            got = run_cut(rp, f"r{k}", toks, cuts)
            assert close(got, want, dtype), (name, graphs, cuts)
            first = got if first is None else first
            assert np.array_equal(got, first), (name, graphs, cuts)
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
    plan = [
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
    solo = replayer(folders[name], dtype, 128)
    for r in toks:
        # (bfloat16: the crowd's bits are those of the request alone, whose closeness to the plain model other tests hold;
        # a short request may be the one row in a hundred whose router picks another expert than the plain model's)
        assert dtype == "bfloat16" or close(np.concatenate(got[r]), want[r], dtype), r
        assert np.array_equal(np.concatenate(got[r]), run_cut(solo, r, toks[r], [lengths[r]])), r
    assert dtype == "float32" or ps.logits_error(np.concatenate(list(np.concatenate(got[r]) for r in toks)),
                                                 np.concatenate([want[r] for r in toks]), quantile=0.5) < 2 * TYPICAL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """300 tokens one by one behind a short prompt, across many pages and partitions of keys: no drift in the states."""
    name = "wide"
    toks = tokens_for(name, 330, 7)
    rp = replayer(folders[name], dtype, 384)
    got = run_cut(rp, "x", toks, [30])
    assert close(got, plain(name, folders[name], toks, dtype), dtype)
    # most of it as one portion (more than 1,024 (row, expert) pairs: the experts' kernel of prompt portions): the same bits
    assert np.array_equal(run_cut(rp, "y", toks, [300]), got)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(folders, dtype):
    """bw.generate with the engine's scheduler, a small token budget and a small page pool: the tokens of the plain
    implementation, which recomputes the whole sequence for every token; crowded and alone give the same bits."""
    name = "mixed"
    cfg, w = CONFIGS[name], weights(folders[name])
    model = bw.Model.load(folders[name], dtype)
    prompts = [tokens_for(name, n, 40 + n) for n in (1, 6, 19, 40)]
    sp = bw.SamplingParams(max_new_tokens=10, ignore_eos=True)
    results = bw.generate(model, prompts, sp, bw.EngineConfig(num_blocks=16, max_batched_tokens=24, max_num_seqs=3, dtype=dtype))
    for p, r in zip(prompts, results):
        assert r.finished and len(r.tokens) == 10
        if dtype == "float32":
            assert r.tokens == ps.generate_greedy(cfg, w, p, 10)
    for p, r in zip(prompts, results):
        solo = bw.generate(model, [p], sp, bw.EngineConfig(num_blocks=16, max_num_seqs=1, dtype=dtype, use_graphs=False))[0]
        assert solo.tokens == r.tokens and solo.logits_fingerprint == r.logits_fingerprint


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_randomized_scenarios_to_the_last_bit(gpu, dtype):
    """The scenario simulator on the architecture's tiny model: every request against its solo run, no wrong token, no
    other logits, no page or slot lost; preemption happens on the way and restarts from zeroed state."""
    from bitwise_amd.registry import ARCHITECTURES
    from bitwise_amd.sim import Simulator

    model = bw.Model.random(ARCHITECTURES["Sepedra"].tiny_config, 43, dtype, sigma=0.08)
    tally = Simulator(model, dtype).run(12, seed=2)
    print(tally.line(dtype))
    assert tally.violations() == 0, "\n".join(tally.notes[:10])
    assert tally.requests_compared > 30 and tally.prefix_hit_tokens == 0


def test_the_recurrence_remembers_the_first_token(folders):
    """A recurrent layer whose decays are pushed towards 1: the first token still moves the logits 200 tokens later,
    through a prompt and through single tokens alike (a state that is dropped or zeroed shows)."""
    from safetensors.torch import load_file, save_file
    name = "only_rglru"
    src = Path(folders[name])
    dst = src.parent / "rglru_long_memory"
    dst.mkdir(exist_ok=True)
    w = load_file(str(src / "model.safetensors"))
    w["l0.mix.lam"] = torch.full_like(w["l0.mix.lam"], -7.0)         # softplus(-7) = 9e-4: a = exp(-8 r 9e-4) > 0.99
    save_file(w, str(dst / "model.safetensors"))
    (dst / "config.json").write_text((src / "config.json").read_text())
    toks = tokens_for(name, 200, 9)
    other = [(toks[0] + 1) % CONFIGS[name]["vocab"]] + toks[1:]
    cfg, w64 = CONFIGS[name], ps.to64(w)
    want, want_other = ps.forward(cfg, w64, toks).numpy(), ps.forward(cfg, w64, other).numpy()
    assert ps.logits_error(want_other[-1:], want[-1:]) > 1e-3, "the first token was meant to matter at the end"
    rp = replayer(dst, "float32", 256)
    for cuts in ([200], [3], [64, 64, 64]):
        assert ps.logits_error(run_cut(rp, "m", toks, cuts), want) < TOL["float32"]
        assert ps.logits_error(run_cut(rp, "o", other, cuts), want_other) < TOL["float32"]


# ----------------------------------------------------------------------------- kernels alone

def _seq_arrays(dev, portions, slots):
    """seq_rows, slots, positions (only their signs matter here) for requests with the given rows in this step."""
    first, rec = 0, []
    for n in portions:
        rec += [first, n]
        first += n
    return (torch.tensor(rec, dtype=torch.int32, device=dev), torch.tensor(slots, dtype=torch.int32, device=dev),
            torch.zeros(max(first, 1), dtype=torch.int32, device=dev), first)


@pytest.mark.parametrize("taps", [1, 2, 3, 4, 6])
def test_causal_conv_through_portions_and_slots(gpu, taps):
    """Two requests convolved in portions of unequal sizes (down to one row, shorter than the taps' reach) in slots that
    a third request then takes over from zero: every row as in one pass over the whole sequence."""
    from bitwise_amd.csrc import ops
    g = torch.Generator().manual_seed(taps)
    C, n = 70, 57
    w = torch.randn(C, taps, generator=g)
    b = torch.randn(C, generator=g)
    xs = [torch.randn(n, C, generator=g) for _ in range(3)]
    want = [ps.causal_conv(x.double(), w.double(), b.double()) for x in xs]
    state = torch.zeros(3, (taps - 1) * C + 5, device=gpu)[:, 5:] if taps > 1 else None          # a view inside a wider slot
    cuts = [[1, 1, 2, 33, 1, 19], [40, 2, 1, 1, 13]]
    got = [[], []]
    at = [0, 0]
    for step in range(max(len(c) for c in cuts)):
        live = [r for r in (0, 1) if step < len(cuts[r])]
        portions = [cuts[r][step] for r in live]
        seq_rows, slots, positions, rows = _seq_arrays(gpu, portions, [2 - r for r in live])
        x = torch.cat([xs[r][at[r]:at[r] + cuts[r][step]] for r in live]).to(gpu)
        out = torch.zeros(rows, C, device=gpu)
        ops.causal_conv(x, w.to(gpu), b.to(gpu), state, seq_rows, slots, positions, len(live), max(portions), out)
        o = 0
        for r in live:
            got[r].append(out[o:o + cuts[r][step]].cpu())
            o += cuts[r][step]
            at[r] += cuts[r][step]
    for r in (0, 1):
        assert (torch.cat(got[r]).double() - want[r]).abs().max() < 1e-5
    if taps > 1:
        state[2].zero_()                   # what the engine does when a request takes a slot
    seq_rows, slots, positions, rows = _seq_arrays(gpu, [n], [2])
    out = torch.zeros(n, C, device=gpu)
    ops.causal_conv(xs[2].to(gpu), w.to(gpu), b.to(gpu), state, seq_rows, slots, positions, 1, n, out)
    assert (out.cpu().double() - want[2]).abs().max() < 1e-5


def test_stretched_frequencies_and_pair_rotation(gpu):
    """The rotary tables against the plain frequencies in all three bands, and the rotation of pairs with the unit norm,
    heads padded to the cache's head size, for a partly rotated head."""
    from bitwise_amd.csrc import ops
    from bitwise_amd.parts.rope import PairRotaryTable
    from bitwise_amd.runtime import Runtime
    r = {"base": 2000.0, "dims": 20, "scaling": {"factor": 5.0, "low": 1.0, "high": 8.0, "original": 96}}
    f = ps.rotary_frequencies(r)
    wl = 2 * np.pi / np.array([2000.0 ** (-2.0 * i / 20) for i in range(10)])
    assert (wl < 96 / 8).any() and (wl > 96).any() and ((wl >= 12) & (wl <= 96)).any(), "all three bands were meant to occur"
    table = PairRotaryTable({"base": r["base"], "dims": r["dims"], "scaling": r["scaling"], "max_positions": 600}, Runtime("float32", gpu))
    assert np.allclose(table.frequencies(), f.numpy(), rtol=1e-14)
    cos, sin = table.tables()
    heads, kv, dim, vdim, hd, page = 3, 1, 28, 12, 32, 8
    g = torch.Generator().manual_seed(4)
    pos = [0, 1, 77, 599]
    src = torch.randn(len(pos), heads * dim + kv * (dim + vdim), generator=g)
    q = torch.zeros(len(pos), heads * hd, device=gpu)
    kc = torch.full((80, kv * page * hd), float("nan"), device=gpu)
    vc = torch.full((80, kv * page * hd), float("nan"), device=gpu)
    table_rows = torch.arange(75, dtype=torch.int32, device=gpu).view(1, -1) + 3
    ops.pair_rope_unit(src.to(gpu), torch.tensor(pos, dtype=torch.int32, device=gpu), torch.zeros(len(pos), dtype=torch.int32, device=gpu),
                       table_rows, cos, sin, q, kc, vc, len(pos), heads, kv, dim, vdim, hd, 20, page, True, 1e-3, True, True)
    for i, p in enumerate(pos):
        qh = src[i:i + 1, :heads * dim].double().view(1, heads, dim)
        want = ps.rms_unit(ps.rotate_pairs(qh, p, r), 1e-3)[0]
        got = q[i].cpu().double().view(heads, hd)
        assert (got[:, :dim] - want).abs().max() < 2e-6 and got[:, dim:].abs().max() == 0
        kh = src[i:i + 1, heads * dim:heads * dim + dim].double().view(1, 1, dim)
        wantk = ps.rms_unit(ps.rotate_pairs(kh, p, r), 1e-3)[0, 0]
        slot = kc[3 + p // page].view(kv, page, hd)[0, p % page].cpu().double()
        assert (slot[:dim] - wantk).abs().max() < 2e-6 and slot[dim:].abs().max() == 0
        vslot = vc[3 + p // page].view(kv, page, hd)[0, p % page].cpu()
        assert torch.equal(vslot[:vdim], src[i, heads * dim + dim:]) and vslot[vdim:].abs().max() == 0


def test_routing_by_groups(gpu):
    """The router's choice against the plain one for several shapes: more experts than lanes, one group, every group
    kept, one expert a row; and a row made so that the best experts outside the kept groups are passed over."""
    from bitwise_amd.csrc import ops
    g = torch.Generator().manual_seed(8)
    for experts, top, count, keep in ((20, 3, 5, 2), (72, 6, 8, 3), (5, 1, 1, 1), (6, 6, 3, 3), (130, 8, 10, 2)):
        z = torch.randn(33, experts, generator=g) * 2
        z[0] = 0.0
        z[0, experts - 1] = 5.0                       # the last group holds the best expert ...
        z[0, 0] = 4.0                                 # ... the first the second best
        mlp = {"router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}
        w = {"mlp.router": torch.eye(experts, dtype=torch.float64)}
        idx, wt = ps.route(z.double(), w, "", mlp)
        ids = torch.zeros(33, top, dtype=torch.int32, device=gpu)
        wts = torch.zeros(33, top, device=gpu)
        ops.moe_route(z.to(gpu), 33, top, count, keep, ids, wts)
        rows = [r for r in range(1, 33)]              # (row 0 has ties among its zeros: the plain top-k may order them otherwise)
        assert torch.equal(ids.cpu().long()[rows], idx[rows]), (experts, top, count, keep)
        assert (wts.cpu().double()[rows] - wt[rows]).abs().max() < 1e-6
        assert int(ids[0, 0]) == experts - 1 and (top == 1 or count == 1 or keep < 2 or int(ids[0, 1]) == 0)


@pytest.mark.parametrize("rows", [150, 700])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_experts_products_over_a_plan(gpu, dtype, rows):
    """Rows dealt to experts very unevenly (one expert gets most rows, some get none): every (row, choice) pair gets its
    own expert's product, whatever tile it lands in; a row alone gets the same bits as in the crowd.  150 rows run the
    kernel of steps with few (row, choice) pairs, 700 rows the one of prompt portions, whose tiles go through LDS; a row
    alone always runs the first, so the two kernels must agree to the last bit.  The inner sizes are no multiples of a
    step."""
    from bitwise_amd.csrc import ops
    g = torch.Generator().manual_seed(9)
    E, top, K, ff = 7, 2, 72, 40
    wg = (torch.randn(E, 2 * ff, K, generator=g) * 0.2).to(dtype)
    wd = (torch.randn(E, K, ff, generator=g) * 0.2).to(dtype)
    x = torch.randn(rows, K, generator=g).to(dtype)
    ids = torch.where(torch.rand(rows, top, generator=g) < 0.7, torch.tensor(3), torch.randint(0, E - 1, (rows, top), generator=g)).int()
    ids[:, 1] = (ids[:, 0] + 1 + ids[:, 1] % (E - 2)) % (E - 1)       # two different experts a row, never the last one
    wts = torch.rand(rows, top, generator=g)

    def run(xr, idr, wtr):
        n = xr.shape[0]
        slots = n * top
        dev = dict(device=gpu)
        srt, place = (torch.zeros(slots, dtype=torch.int32, **dev) for _ in range(2))
        tiles = torch.zeros(4 * ops.moe_max_tiles(slots, E), dtype=torch.int32, **dev)
        meta = torch.zeros(4, dtype=torch.int32, **dev)
        ops.moe_plan(idr.to(gpu).contiguous(), slots, E, srt, place, tiles, meta)
        act = torch.zeros(slots, ff, dtype=dtype, **dev)
        ops.moe_experts(xr.to(gpu), wg.to(gpu), act, srt, tiles, meta, slots, top, True, 0.8, 1.702)
        y = torch.zeros(slots, K, **dev)
        ops.moe_experts(act, wd.to(gpu), y, srt, tiles, meta, slots, top, False)
        out = torch.zeros(n, K, **dev)
        ops.moe_combine(y, place, wtr.to(gpu).contiguous(), top, out, n, False)
        return out.cpu()

    got = run(x, ids, wts)
    rnd = ps.round_bf16 if dtype == torch.bfloat16 else ps.identity
    w = {}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = wg[e, :ff].double(), wg[e, ff:].double(), wd[e].double()
    want = torch.zeros(rows, K, dtype=torch.float64)
    for r in range(rows):
        for j in range(top):
            want[r] += wts[r, j].double() * ps.expert(x[r:r + 1].double(), w, f"e{int(ids[r, j])}", 0.8, rnd)[0]
    assert (got.double() - want).abs().max() < (2e-5 if dtype == torch.float32 else 2e-2) * want.abs().max()
    for r in (0, 77, rows - 1):
        assert torch.equal(run(x[r:r + 1], ids[r:r + 1], wts[r:r + 1])[0], got[r])


def _fill_caches(keys, values, kv_heads, hd, page, dtype, dev):
    """Caches of one request whose pages lie scattered: keys [n, kv_heads, hd], values likewise."""
    n = keys.shape[0]
    pages = (n + page - 1) // page
    order = torch.randperm(pages + 3, generator=torch.Generator().manual_seed(3))[:pages]
    kc = torch.full((pages + 3, kv_heads * page * hd), float("nan"), dtype=dtype)
    vc = torch.full((pages + 3, kv_heads * page * hd), float("nan"), dtype=dtype)
    pk_ = torch.zeros(pages * page, kv_heads, hd, dtype=torch.float64)
    pv_ = torch.zeros(pages * page, kv_heads, hd, dtype=torch.float64)
    pk_[:n], pv_[:n] = keys, values
    for i in range(pages):
        kp = pk_[i * page:(i + 1) * page].permute(1, 0, 2)                      # [kv head][slot][element]
        vp = pv_[i * page:(i + 1) * page].permute(1, 0, 2)
        kc[order[i]] = kp.reshape(-1).to(dtype)
        vc[order[i]] = (vp.transpose(1, 2) if dtype == torch.bfloat16 else vp).reshape(-1).to(dtype)   # bfloat16 values: [kv head][element][slot]
    return kc.to(dev), vc.to(dev), order.to(torch.int32).view(1, -1).to(dev)


def _plain_attention(q, keys, values, heads, kv_heads, scale, positions, sink):
    out = torch.zeros(len(positions), heads, values.shape[-1], dtype=torch.float64)
    for r, p in enumerate(positions):
        for h in range(heads):
            kvh = h // (heads // kv_heads)
            s = (keys[:p + 1, kvh] @ q[r, h]) * scale
            if sink is not None:
                s = torch.cat([s, sink[h:h + 1]])
            wgt = torch.softmax(s, -1)
            out[r, h] = wgt[:p + 1] @ values[:p + 1, kvh]
    return out


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds_page_borders_and_the_sink(gpu, dtype):
    """Every probe's query is a scaled copy of one key far back (the first, keys beside a page's and a partition's
    border, the one before the last), so that this key carries the softmax: a key that is lost or read from a wrong
    slot shows.  With a sink of score 0 the weights no longer sum to one, a large sink leaves little for the values,
    a very negative one changes nothing; through the kernels of prompt portions and of decoded tokens alike."""
    from bitwise_amd.csrc import ops
    g = torch.Generator().manual_seed(5)
    heads, kv, hd, page, n = 4, 2, 48, 16, 700
    keys = torch.randn(n, kv, hd, generator=g, dtype=torch.float64)
    keys = keys / keys.pow(2).mean(-1, keepdim=True).sqrt()
    values = torch.randn(n, kv, hd, generator=g, dtype=torch.float64)
    if dtype == torch.bfloat16:
        keys, values = keys.bfloat16().double(), values.bfloat16().double()
    targets = [0, 1, 15, 16, 17, 63, 64, 65, 300, 511, 512, 640, 698, 699]
    early = [0, 1, 5]                                       # and queries with one, two and six keys, where a sink weighs most
    positions = [n - 1] * len(targets) + early
    q = torch.randn(len(positions), heads, hd, generator=g, dtype=torch.float64) * 0.1
    for r, t in enumerate(targets):
        q[r, r % heads] += 1.0 * keys[t, (r % heads) // (heads // kv)]
    if dtype == torch.bfloat16:
        q = q.bfloat16().double()
    kc, vc, table = _fill_caches(keys, values, kv, hd, page, dtype, gpu)
    rows = len(positions)
    pos = torch.tensor(positions, dtype=torch.int32, device=gpu)
    row_seq = torch.zeros(rows, dtype=torch.int32, device=gpu)
    tiles = torch.tensor([[r, 1, 0, 0] for r in range(rows)], dtype=torch.int32, device=gpu)
    qd = q.reshape(rows, heads * hd).to(dtype).to(gpu).contiguous()
    tol = 2e-5 if dtype == torch.float32 else 1.5e-2
    for sink in (None, torch.zeros(heads), torch.tensor([9.0, 0.0, -30.0, 2.0])):
        want = _plain_attention(q, keys, values, heads, kv, 0.25, positions, None if sink is None else sink.double())
        sk = None if sink is None else sink.to(gpu)
        routes = []
        if dtype == torch.float32:
            out = torch.zeros(rows, heads * hd, device=gpu)
            ops.attention_f32(qd, pos, row_seq, table, kc, vc, out, rows, heads, kv, hd, page, 0, 0.25, sink=sk)
            routes.append(("rows", out))
            for tiled in (1, 2, False):
                out = torch.zeros(rows, heads * hd, device=gpu)
                ops.attention_f32_tiles(qd, pos, table, tiles, rows, tiled, kc, vc, out, heads, kv, hd, page, 0, 0.25, sink=sk)
                routes.append((f"tiles {tiled}", out))
        else:
            group = ops.fold_group_tiles(hd)
            padded = torch.tensor([[r, 1, 0, 0] for r in range(rows)] + [[0, 0, 0, 0]] * (-rows % group), dtype=torch.int32, device=gpu)
            out = torch.zeros(rows, heads * hd, dtype=dtype, device=gpu)
            ops.attention_bf16(qd, pos, table, padded, padded.shape[0], kc, vc, out, heads, kv, hd, page, 0, 0.25, sink=sk)
            routes.append(("fold", out))
            out = torch.zeros(rows, heads * hd, dtype=dtype, device=gpu)
            ops.attention_bf16(qd, pos, table, tiles, rows, kc, vc, out, heads, kv, hd, page, 0, 0.25, decode=True, sink=sk)
            routes.append(("decode", out))
        for what, out in routes:
            got = out.cpu().double().view(rows, heads, hd)
            assert (got - want).abs().max() < tol * want.abs().max(), (what, sink)
            assert torch.equal(out, routes[0][1]), (what, "the routes were meant to give the same bits")
        if sink is None:
            for r, t in enumerate(targets):       # the probe's head returns (nearly) the value of its target
                h = r % heads
                assert (want[r, h] - values[t, h // (heads // kv)]).abs().max() < 0.1, t
            plain_none = want
        elif float(sink.abs().max()) == 0:
            # the first token's only key shares the weight with the sink: about half of its value is left
            assert (want[len(targets)] - plain_none[len(targets)]).abs().max() > 0.2
        else:
            quiet = [r for r in range(rows) if r % heads != 0 or r >= len(targets)]      # rows whose head 0 has no key that stands out
            assert want[quiet, 0].abs().max() < 0.5 * plain_none[quiet, 0].abs().max()
            assert (want[:, 2] - plain_none[:, 2]).abs().max() < 1e-6
