"""The Potatar decoder through the engine (model registry, loader, cache and state manager, step function,
scheduler, entry point) against the plain implementation, in every cutting of the requests."""
import json

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import potatar_plain as N
import traces
from potatar_tiny import PA, TINY, attention, ff, make_folder, parallel, random_tensors, wkv, write_folder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("potatar")
    return {which: make_folder(tmp, which) for which in TINY}


def _requests(vocab, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {f"q{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def _reference(folder, reqs):
    cfg, w = N.read_folder(folder)
    return {rid: N.forward(cfg, w, toks).float() for rid, toks in reqs.items()}


def _tail_cut(reqs, tail=20):
    """All but the last ``tail`` tokens in one step (at least one), the rest one by one."""
    t = traces.Trace()
    for rid, toks in reqs.items():
        n = max(1, len(toks) - tail)
        t.step([(rid, toks[:n])], end=[rid] if n == len(toks) else [])
        for i in range(n, len(toks)):
            t.step([(rid, toks[i:i + 1])], end=[rid] if i == len(toks) - 1 else [])
    return t


def _one_by_one(reqs):
    """Every token a step of its own, from the first: nothing but the decoding path."""
    t = traces.Trace()
    for rid, toks in reqs.items():
        for i in range(len(toks)):
            t.step([(rid, toks[i:i + 1])], end=[rid] if i == len(toks) - 1 else [])
    return t


CUTS = {"whole": traces.whole, "tail": _tail_cut, "portions": traces.portions, "mixed": lambda r: traces.mixed(r, seed=3),
        "twos": lambda r: traces.portions(r, sizes=(2,)), "ones": _one_by_one}


def _errors(got, ref):
    out = []
    for rid, rows in ref.items():
        scale = float(rows.abs().max())
        out += [float((torch.from_numpy(got[rid][p]) - rows[p]).abs().max()) / scale for p in range(rows.shape[0])]
    return torch.tensor(out)


def _assert_bfloat16_close(got, ref, what, median=2e-2, largest=1.2e-1):
    err = _errors(got, ref)
    assert not torch.isnan(err).any(), what
    assert float(err.median()) < median, f"{what}: median error {float(err.median())}"
    assert float(err.max()) < largest, f"{what}: largest error {float(err.max())}"


@pytest.mark.parametrize("cut", sorted(CUTS))
@pytest.mark.parametrize("which", sorted(TINY))
def test_every_cutting_in_float32(folders, tmp_path, which, cut):
    cfg, _, page = TINY[which]
    lengths = (70, 33, 121, 58, 2, 95) if cut != "ones" else (45, 2, 30)
    reqs = _requests(cfg["vocab"], lengths, seed=7)
    ref = _reference(folders[which], reqs)
    trace = CUTS[cut](reqs)
    out = str(tmp_path / "out")
    traces.run_in_process(trace, folders[which], "float32", out, page)
    got = traces.collect(trace, out, cfg["vocab"])
    bad, worst = traces.first_mismatch(got, ref, 2e-4)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"


@pytest.mark.parametrize("which", sorted(TINY))
def test_bfloat16_agrees_with_the_plain_model_and_with_itself_in_every_cutting(folders, tmp_path, which):
    cfg, _, page = TINY[which]
    reqs = _requests(cfg["vocab"], (70, 33, 121, 58), seed=8)
    ref = _reference(folders[which], reqs)
    got = {}
    for cut in ("whole", "mixed", "portions", "tail"):
        trace = CUTS[cut](reqs)
        out = str(tmp_path / cut)
        traces.run_in_process(trace, folders[which], "bfloat16", out, page)
        got[cut] = traces.collect(trace, out, cfg["vocab"])
        # (with alpha 1 a mixer's rounding weighs as much as the stream: twice the allowance against 64-bit)
        _assert_bfloat16_close(got[cut], ref, f"{cut} against the plain model", median=4e-2, largest=5e-1)
    whole = {rid: torch.stack([torch.from_numpy(got["whole"][rid][p]) for p in range(len(t))]) for rid, t in reqs.items()}
    for cut in ("mixed", "portions", "tail"):
        _assert_bfloat16_close(got[cut], whole, f"{cut} against whole prompts")


def test_the_program_replays_a_trace(folders, tmp_path):
    """bin/trace_run as a user starts it, steps going in one at a time."""
    cfg, _, page = TINY["A"]
    reqs = _requests(cfg["vocab"], (40, 9, 27), seed=5)
    ref = _reference(folders["A"], reqs)
    trace = traces.mixed(reqs, seed=1)
    out = str(tmp_path / "out")
    traces.run_program(trace, folders["A"], "float32", out, page)
    bad, worst = traces.first_mismatch(traces.collect(trace, out, cfg["vocab"]), ref, 2e-4)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"


def test_long_decoding_over_many_pages_and_chunks(folders, tmp_path):
    """Five tokens of prompt, then one at a time through dozens of chunks and pages: the recurrences' states are
    carried for hundreds of steps, every chunk's first and last position is a decoded token."""
    cfg, _, page = TINY["A"]
    reqs = _requests(cfg["vocab"], (330,), seed=9)
    ref = _reference(folders["A"], reqs)
    trace = traces.tail_decoded(reqs, tail=325)
    out = str(tmp_path / "out")
    traces.run_in_process(trace, folders["A"], "float32", out, page)
    bad, worst = traces.first_mismatch(traces.collect(trace, out, cfg["vocab"]), ref, 2e-4)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"


def test_hundreds_of_keys_in_one_chunk(folders, tmp_path):
    """Chunks longer than the sequences: the last positions see several hundred keys over many pages, in prompts cut
    into portions and decoded one by one."""
    cfg, _, page = TINY["C"]
    reqs = _requests(cfg["vocab"], (700, 333), seed=10)
    ref = _reference(folders["C"], reqs)
    for cut, trace in (("whole", traces.whole(reqs)), ("tail", traces.tail_decoded(reqs, tail=40)),
                       ("portions", traces.portions(reqs, sizes=(190, 2, 64, 301, 5)))):
        out = str(tmp_path / cut)
        traces.run_in_process(trace, folders["C"], "float32", out, page)
        bad, worst = traces.first_mismatch(traces.collect(trace, out, cfg["vocab"]), ref, 2e-4)
        assert bad is None, f"{cut}: first wrong logits at (request, position, relative error) {bad}"


# ---- a chunk's edges ---------------------------------------------------------------------------------------------
def _one_layer(kind, size, seed=41):
    """One layer without a feed-forward: what its last query sees or does not see decides its logits, since nothing
    else carries a token's identity forward (the linear half beside the biased attention forgets at once: decay 0)."""
    if kind == "attention":
        layer = attention(4, 2, 12, 20, size, 4, 0.6, True, 1000.0, None)
        sizes = {}
    else:
        layer = parallel(6, 3, 8, size, 0.7, 3.0 * size, 2, 12, 8, (0.0, 0.0), 0.9, 1.1, None)
        sizes = {0: 10}
    cfg = dict(PA, layers=[layer])
    return cfg, random_tensors(cfg, seed, torch.float32, sizes)


@pytest.mark.parametrize("kind", ["attention", "parallel"])
@pytest.mark.parametrize("size,page", [(16, 8), (17, 8), (5, 4), (33, 16), (64, 16), (100, 16)])
def test_keys_just_inside_and_just_outside_a_chunk(tmp_path, kind, size, page):
    """Changing one token changes the logits of later positions exactly where the plain model says: the first
    position of the last query's chunk is seen, the position before it is not, and the chunk's last query sees
    the whole chunk.  Prompts, portions and single decoded tokens alike, with chunk edges on and beside page borders."""
    cfg, w = _one_layer(kind, size)
    folder = write_folder(str(tmp_path / "model"), cfg, w)
    cfg_, w_ = N.read_folder(folder)
    g = torch.Generator().manual_seed(size)
    n = 3 * size + size // 2 + 1                   # the last query sits in the middle of the fourth chunk
    base = torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
    first = (n - 1) // size * size
    reqs = {"base": base}
    for name, p in (("in", first), ("out", first - 1), ("far", 0)):
        other = list(base)
        other[p] = (base[p] + 1) % cfg["vocab"]
        reqs[name] = other
    ref = {rid: N.forward(cfg_, w_, toks).float() for rid, toks in reqs.items()}
    last = ref["base"][-1]
    scale = float(last.abs().max())
    assert float((ref["in"][-1] - last).abs().max()) > 1e-4 * scale            # the chunk's first key is seen
    assert float((ref["out"][-1] - last).abs().max()) < 1e-7 * scale           # the key before it is not
    assert float((ref["far"][-1] - last).abs().max()) < 1e-7 * scale
    # the last position of the third chunk sees that chunk's first key, the position after it does not
    end = first - 1
    other = list(base)
    other[first - size] = (base[first - size] + 1) % cfg["vocab"]
    reqs["third"] = other
    ref["third"] = N.forward(cfg_, w_, other).float()
    assert float((ref["third"][end] - ref["base"][end]).abs().max()) > 1e-4 * scale
    assert float((ref["third"][end + 1] - ref["base"][end + 1]).abs().max()) < 1e-7 * scale
    for cut, trace in (("whole", traces.whole(reqs)), ("tail", traces.tail_decoded(reqs, tail=size + size // 2 + 3)),
                       ("portions", traces.portions(reqs)), ("mixed", traces.mixed(reqs, seed=size))):
        out = str(tmp_path / cut)
        traces.run_in_process(trace, folder, "float32", out, page)
        got = traces.collect(trace, out, cfg["vocab"])
        bad, worst = traces.first_mismatch(got, ref, 2e-5)       # (well below what one key more or less changes)
        assert bad is None, f"{cut}: first wrong logits at (request, position, relative error) {bad}"


def test_the_first_tokens_of_a_sequence(tmp_path):
    """The token before the first one is zeros for the blends, the states start from zero, position 0 turns nothing:
    the first three positions' logits, alone and with the rest, in all four layer orders that start differently."""
    for i, first in enumerate((wkv(3, 8, ff(24)), attention(4, 2, 12, 20, 13, 4, 0.3, True, 1000.0, None),
                               parallel(6, 3, 8, 21, 0.35, 30, 2, 12, 8, (0.5, 0.93), 0.7, 1.3, None))):
        cfg = dict(PA, layers=[first, wkv(2, 4, None)])
        sizes = {0: 5 if first["type"] == "wkv" else 10, 1: 3}
        folder = write_folder(str(tmp_path / f"m{i}"), cfg, random_tensors(cfg, 50 + i, torch.float32, sizes))
        cfg_, w_ = N.read_folder(folder)
        reqs = _requests(cfg["vocab"], (1, 2, 3, 9), seed=i)
        ref = {rid: N.forward(cfg_, w_, toks).float() for rid, toks in reqs.items()}
        for cut in ("whole", "ones", "mixed"):
            trace = CUTS[cut](reqs)
            out = str(tmp_path / f"o{i}{cut}")
            traces.run_in_process(trace, folder, "float32", out, 4)
            bad, worst = traces.first_mismatch(traces.collect(trace, out, cfg["vocab"]), ref, 1e-4)
            assert bad is None, f"{first['type']} first, {cut}: {bad}"


@pytest.mark.parametrize("kind", ["wkv", "attention", "parallel"])
def test_models_of_one_kind_of_layer(tmp_path, kind):
    """Nothing but recurrences (no keys are cached at all), nothing but attention (no state), nothing but the two
    side by side: two layers each, in every cutting."""
    layer = {"wkv": wkv(2, 12, ff(40)), "attention": attention(4, 2, 12, 20, 13, 4, 0.3, True, 1000.0, ff(48)),
             "parallel": parallel(6, 3, 8, 21, 0.35, 30, 2, 12, 8, (0.5, 0.93), 0.7, 1.3, None)}[kind]
    cfg = dict(PA, layers=[layer, layer])
    sizes = {0: 7, 1: 7} if kind == "wkv" else {0: 10, 1: 10}
    folder = write_folder(str(tmp_path / "model"), cfg, random_tensors(cfg, 77, torch.float32, sizes))
    cfg_, w_ = N.read_folder(folder)
    reqs = _requests(cfg["vocab"], (50, 3, 29), seed=6)
    ref = {rid: N.forward(cfg_, w_, toks).float() for rid, toks in reqs.items()}
    for cut in ("whole", "mixed", "ones"):
        trace = CUTS[cut](reqs)
        out = str(tmp_path / cut)
        traces.run_in_process(trace, folder, "float32", out, 8)
        bad, worst = traces.first_mismatch(traces.collect(trace, out, cfg["vocab"]), ref, 2e-4)
        assert bad is None, f"{cut}: first wrong logits at (request, position, relative error) {bad}"


# ---- slots and pages -----------------------------------------------------------------------------------------------
def test_slots_and_pages_that_come_back_start_clean(folders):
    """A request that takes over the state slot and the pages of one that ended computes what it computes alone: the
    recurrences start from zero, the token before its first is zeros, no old key is seen."""
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    cfg, _, page = TINY["A"]
    reqs = _requests(cfg["vocab"], (40, 37), seed=11)
    ref = _reference(folders["A"], reqs)
    runner = ModelRunner(load_model(folders["A"], dtype="float32"), page_size=page, num_pages=6, max_requests=1,
                         debug_poison=True)
    for rid in ("q0", "q1", "q0"):
        toks = reqs[rid]
        runner.add_request(rid)
        a = runner.step([StepEntry(rid, toks[:5], [4])])
        b = runner.step([StepEntry(rid, toks[5:], list(range(len(toks) - 5)))])
        runner.free_request(rid)
        runner.cache.check_invariants()
        got = torch.cat([a, b]).cpu()
        err = float((got - ref[rid][4:]).abs().max()) / float(ref[rid].abs().max())
        assert err < 2e-4, f"{rid}: {err}"


def test_four_slots_shared_by_many_requests(folders, tmp_path):
    """Ten unequal requests through four slots and a pool for the live ones only."""
    cfg, _, page = TINY["B"]
    reqs = _requests(cfg["vocab"], (64, 3, 90, 17, 128, 41, 2, 77, 130, 25), seed=21)
    ref = _reference(folders["B"], reqs)
    trace = traces.mixed(reqs, seed=4, max_live=4, tail=9)
    assert trace.max_tokens < sum(traces.round64(len(t)) for t in reqs.values())
    out = str(tmp_path / "out")
    traces.run_in_process(trace, folders["B"], "float32", out, page)
    bad, worst = traces.first_mismatch(traces.collect(trace, out, cfg["vocab"]), ref, 2e-4)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"


# ---- generation ----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B"])
def test_greedy_generation_through_the_entry_point(folders, dtype, which):
    from qwen_engine_amd import EngineConfig, SamplingParams, generate
    cfg, _, page = TINY[which]
    cfg_, w_ = N.read_folder(folders[which])
    prompts = list(_requests(cfg["vocab"], (19, 3, 44), seed=12).values())
    res = generate(folders[which], prompts, SamplingParams(max_new_tokens=12, ignore_eos=True),
                   EngineConfig(dtype=dtype, block_size=page, max_num_seqs=2, max_model_len=64, max_step_tokens=32,
                                prefill_chunk=8, debug_poison=True))
    for prompt, r in zip(prompts, res):
        assert r.finish_reason == "length" and len(r.token_ids) == 12
        logits = N.forward(cfg_, w_, prompt + r.token_ids[:-1]).float()
        for i, tok in enumerate(r.token_ids):
            row = logits[len(prompt) - 1 + i]
            if dtype == "float32":
                assert tok == int(row.argmax()), f"token {i} of a prompt of {len(prompt)}"
            else:
                assert float(row.max() - row[tok]) <= 4e-2 * float(row.abs().max()), f"token {i} of a prompt of {len(prompt)}"


def test_recorded_decode_steps_give_the_tokens_of_steps_run_as_they_come(folders):
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    cfg, _, page = TINY["B"]
    model = load_model(folders["B"], dtype="bfloat16")
    prompts = list(_requests(cfg["vocab"], (21, 9, 30), seed=13).values())
    outs = []
    for use_graphs in (False, True):
        runner = ModelRunner(model, page_size=page, num_pages=24, max_requests=3, use_graphs=use_graphs)
        last = []
        for i, p in enumerate(prompts):
            runner.add_request(i)
            last.append(runner.step([StepEntry(i, p, [len(p) - 1])], greedy=True)[0])
        rows = [list(last)]
        for _ in range(30):                       # (past the ends of chunks of 40 positions)
            last = runner.step([StepEntry(i, [last[i]], [0]) for i in range(3)], greedy=True)
            rows.append(list(last))
        outs.append(rows)
        if use_graphs:
            assert runner.graph_steps_of["decode"] == 30
    assert outs[0] == outs[1]


def test_command_line_with_random_weights(tmp_path, capsys):
    """main.py writes random weights for a Potatar config.json and generates from token ids."""
    import main as cli
    cfg, _, page = TINY["B"]
    d = json.loads(json.dumps(cfg))
    d["layers"][0]["mixer"]["left"]["bias_rows"] = 14           # what no tensor's shape can give yet
    d["layers"][2]["mixer"]["decay_rank"] = 24
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(d))
    folder = str(tmp_path / "model")
    rc = cli.main(["--model-name-or-path", folder, "--random-weights", str(cfg_path), "--seed", "3", "--prompt-ids", "5,17,3",
                   "--prompt-ids", "9,9,200,41", "--max-new-tokens", "6", "--block-size", str(page), "--max-model-len", "64",
                   "--ignore-eos", "--stats"])
    assert rc == 0
    out = capsys.readouterr().out
    assert out.count("Prompt:") == 2 and "5 17 3" in out
    stats = json.loads(out.strip().splitlines()[-1])
    assert stats["graph_steps_decode"] >= 4                 # single new tokens were replayed from recorded steps
    cfg_, w_ = N.read_folder(folder)
    assert set(w_) == set(random_tensors(cfg, 0))           # every tensor of the design, by its name


# Sizes at which the bfloat16 mode runs the kernels on the matrix units inside the engine, with prompts long enough
# for several key splits of the decode kernels and many tiles of the prefill kernels; chunks that cross many pages
# and tiles and whose edges fall inside them.
PM = {"architecture": "Potatar", "vocab": 701, "width": 320, "norm": {"eps": 1e-5}, "postln_alpha": 2.0, "logit_softcap": 20.0,
      "layers": [
          attention(6, 2, 64, 40, 150, 24, 0.12, True, 20000.0, ff(256)),
          parallel(8, 2, 32, 150, 0.2, 200, 4, 24, 48, (0.7, 0.9, 0.96, 0.998), 1.1, 0.9, ff(128)),
          wkv(5, 64, None),
          attention(4, 2, 128, 40, 333, 128, 0.09, True, 3000.0, ff(192)),
          parallel(3, 1, 64, 70, 0.13, 64, 2, 64, 40, (0.95, 0.5), 0.8, 1.2, None),
      ]}
PM_SIZES = {1: 24, 2: 32, 4: 9}


@pytest.fixture(scope="module")
def medium(tmp_path_factory):
    folder = write_folder(str(tmp_path_factory.mktemp("potatar_m") / "model"), PM, random_tensors(PM, 21, sizes=PM_SIZES))
    reqs = _requests(PM["vocab"], (610, 75, 380), seed=14)
    return folder, reqs, _reference(folder, reqs)


def _medium_mixed(reqs):
    """The long prompt in large portions beside the others' small portions and single tokens."""
    t = traces.Trace()
    a, b, c = reqs["q0"], reqs["q1"], reqs["q2"]
    t.step([("q0", a[:400]), ("q1", b[:3])])
    t.step([("q1", b[3:4]), ("q0", a[400:590]), ("q2", c[:350])])
    t.step([("q2", c[350:352]), ("q1", b[4:5])])
    for i in range(20):
        entries = [("q0", a[590 + i:591 + i]), ("q2", c[352 + i:353 + i])]
        if 5 + i < len(b):
            entries.append(("q1", b[5 + i:6 + i]))
        t.step(entries)
    t.step([("q1", b[25:]), ("q2", c[372:])], end=["q0", "q1", "q2"])
    return t


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "mixed"])
def test_medium_sizes_with_long_prompts(medium, tmp_path, dtype, cut):
    folder, reqs, ref = medium
    trace = traces.whole(reqs) if cut == "whole" else _medium_mixed(reqs)
    out = str(tmp_path / "out")
    traces.run_in_process(trace, folder, dtype, out, 16)
    got = traces.collect(trace, out, PM["vocab"])
    if cut == "mixed":
        ref = {rid: rows[:max(got[rid]) + 1] for rid, rows in ref.items()}
    if dtype == "float32":
        bad, worst = traces.first_mismatch(got, ref, 2e-4)
        assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"
    else:
        _assert_bfloat16_close(got, ref, f"{cut} against the plain model")
