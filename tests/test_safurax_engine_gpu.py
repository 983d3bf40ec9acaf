"""The Safurax decoder through the engine (model registry, loader, cache manager, step function, scheduler, entry
point) against the plain implementation, in every cutting of the requests."""
import copy
import json

import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import safurax_plain as S
import traces
from safurax_tiny import SA, TINY, make_folder, random_config, random_tensors, write_folder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("safurax")
    return {which: make_folder(tmp, which) for which in TINY}


def _requests(vocab, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {f"q{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def _reference(folder, reqs):
    cfg, w = S.read_folder(folder)
    return {rid: S.forward(cfg, w, toks).float() for rid, toks in reqs.items()}


def _tail_cut(reqs, tail=20):
    """All but the last ``tail`` tokens in one step (at least one), the rest one by one."""
    t = traces.Trace()
    for rid, toks in reqs.items():
        n = max(1, len(toks) - tail)
        t.step([(rid, toks[:n])], end=[rid] if n == len(toks) else [])
        for i in range(n, len(toks)):
            t.step([(rid, toks[i:i + 1])], end=[rid] if i == len(toks) - 1 else [])
    return t


CUTS = {"whole": traces.whole, "tail": _tail_cut, "portions": traces.portions, "mixed": lambda r: traces.mixed(r, seed=3)}


def _position_errors(got, ref):
    out = []
    for rid, rows in ref.items():
        scale = float(rows.abs().max())
        out += [float((torch.from_numpy(got[rid][p]) - rows[p]).abs().max()) / scale for p in range(rows.shape[0])]
    return torch.tensor(out)


def _assert_close_but_for_close_calls(got, ref, what):
    """In bfloat16 a router's close call may fall the other way, and then that token's logits (and a little of what
    follows) differ by a choice, not by rounding: the typical position agrees to rounding, few do not, nothing is NaN."""
    err = _position_errors(got, ref)
    assert not torch.isnan(err).any(), what
    assert float(err.median()) < 1.5e-2, f"{what}: median error {float(err.median())}"
    assert float((err > 6e-2).float().mean()) <= 0.06, f"{what}: {int((err > 6e-2).sum())} of {len(err)} positions differ"


@pytest.mark.parametrize("cut", sorted(CUTS))
@pytest.mark.parametrize("which", sorted(TINY))
def test_every_cutting_in_float32(folders, tmp_path, which, cut):
    """Prompts longer than every window of the tiny models (so that pages go back while a request runs), of one
    and of two tokens, in every cutting, with poisoned pages."""
    cfg, _, page = TINY[which]
    reqs = _requests(cfg["vocab"], (70, 33, 121, 58, 2, 95, 1), seed=7)
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
    page = 16 if which in "BD" else page      # (pages of 16: the matrix-unit kernels where the sizes allow them)
    reqs = _requests(cfg["vocab"], (70, 33, 121, 58), seed=8)
    ref = _reference(folders[which], reqs)
    got = {}
    for cut in ("whole", "mixed", "portions"):
        trace = CUTS[cut](reqs)
        out = str(tmp_path / cut)
        traces.run_in_process(trace, folders[which], "bfloat16", out, page)
        got[cut] = traces.collect(trace, out, cfg["vocab"])
        _assert_close_but_for_close_calls(got[cut], ref, f"{cut} against the plain model")
    whole = {rid: torch.stack([torch.from_numpy(got["whole"][rid][p]) for p in range(len(t))]) for rid, t in reqs.items()}
    for cut in ("mixed", "portions"):
        _assert_close_but_for_close_calls(got[cut], whole, f"{cut} against whole prompts")


def test_long_decoding_over_many_pages_and_windows(folders, tmp_path):
    cfg, _, page = TINY["A"]
    reqs = _requests(cfg["vocab"], (340,), seed=9)
    ref = _reference(folders["A"], reqs)
    trace = traces.tail_decoded(reqs, tail=335)               # five tokens of prompt, then one at a time
    out = str(tmp_path / "out")
    traces.run_in_process(trace, folders["A"], "float32", out, page)
    bad, worst = traces.first_mismatch(traces.collect(trace, out, cfg["vocab"]), ref, 2e-4)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"


def _one_layer(kind, tmp_path, name, sharpen, mixer=None):
    """A model of one layer of SA (by its type), with the named tensor scaled so that few keys carry the weight."""
    layer = copy.deepcopy(next(l for l in SA["layers"] if l["type"] == kind and "kv_from" not in l["mixer"]))
    layer["mixer"].update(mixer or {})
    cfg = dict(SA, layers=[layer])
    w = random_tensors(cfg, 31, torch.float32)
    for n, f in sharpen.items():
        w[n] *= f
    return cfg, write_folder(str(tmp_path / name), cfg, w)


@pytest.mark.parametrize("kind,sharpen", [("latent_attention", {"l0.mix.uq": 4.0}), ("attention", {"l0.mix.q.norm": 4.0})])
def test_a_far_token_decides_the_logits(tmp_path, kind, sharpen):
    """One layer with sharp scores: the logits at the end depend on the identity of one early token hundreds of
    positions back, by as much in the engine as in the plain model; a key lost at a page border would show."""
    cfg, folder = _one_layer(kind, tmp_path, "model", sharpen)
    page = 8
    g = torch.Generator().manual_seed(10)
    base = torch.randint(0, cfg["vocab"], (400,), generator=g).tolist()
    cfg_, w_ = S.read_folder(folder)
    ref_a = S.forward(cfg_, w_, base).float()
    moved = {}
    for p in (3, 7, 8, 15, 16, 17, 63, 64):
        other = list(base)
        other[p] = (base[p] + 1) % cfg["vocab"]
        moved[p] = (float((S.forward(cfg_, w_, other).float()[-1] - ref_a[-1]).abs().max()), other)
    p, (delta, other) = max(moved.items(), key=lambda kv: kv[1][0])
    assert delta > 1e-3 * float(ref_a.abs().max())
    reqs = {"a": base, "b": other}
    ref = {"a": ref_a, "b": S.forward(cfg_, w_, other).float()}
    trace = traces.tail_decoded(reqs, tail=40)
    out = str(tmp_path / "out")
    traces.run_in_process(trace, folder, "float32", out, page)
    got = traces.collect(trace, out, cfg["vocab"])
    bad, worst = traces.first_mismatch(got, ref, 1e-4)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"


@pytest.mark.parametrize("window", [37, 16, 3])
def test_a_token_at_the_windows_edge_decides_and_one_behind_it_does_not(tmp_path, window):
    """One windowed layer with sharp scores and sinks far below.  Changing the token at position p changes the logits
    at p + window - 1 (the last position that sees it) and leaves those at p + window exactly as they were, in prompts'
    portions and in decoding, in the engine as in the plain model."""
    cfg, folder = _one_layer("latent_attention_2", tmp_path, "model", {"l0.mix.q": 3.0}, mixer={"mask": {"size": window}})
    page = 8
    g = torch.Generator().manual_seed(11)
    base = torch.randint(0, cfg["vocab"], (130,), generator=g).tolist()
    p = 40
    other = list(base)
    other[p] = (base[p] + 1) % cfg["vocab"]
    cfg_, w_ = S.read_folder(folder)
    ref = {"a": S.forward(cfg_, w_, base).float(), "b": S.forward(cfg_, w_, other).float()}
    last_in, first_out = p + window - 1, p + window
    assert float((ref["a"][last_in] - ref["b"][last_in]).abs().max()) > 1e-5 * float(ref["a"].abs().max())
    assert torch.equal(ref["a"][first_out:], ref["b"][first_out:])
    reqs = {"a": base, "b": other}
    for name, trace in (("portions", traces.portions(reqs)), ("decoded", traces.tail_decoded(reqs, tail=130 - p - 2))):
        out = str(tmp_path / name)
        traces.run_in_process(trace, folder, "float32", out, page)
        got = traces.collect(trace, out, cfg["vocab"])
        bad, worst = traces.first_mismatch(got, ref, 1e-4)
        assert bad is None, f"{name}: first wrong logits at (request, position, relative error) {bad}"
        assert not (got["a"][last_in] == got["b"][last_in]).all()
        for q in range(first_out, 130):
            assert (got["a"][q] == got["b"][q]).all(), f"{name}: position {q} still sees position {p}"


def test_slots_and_pages_that_come_back_start_clean(folders):
    """A request that takes over the pages of one that ended computes what it computes alone."""
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


def test_a_window_gives_its_pages_back_while_the_request_runs(folders):
    """The windowed group of model A keeps the widest window among a layer and the layers that read its cache (50
    keys); a request of 200 tokens never holds more pages of it than that window spans."""
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    cfg, _, page = TINY["A"]
    toks = _requests(cfg["vocab"], (200,), seed=12)["q0"]
    runner = ModelRunner(load_model(folders["A"], dtype="float32"), page_size=page, num_pages=40, max_requests=1)
    runner.add_request("r")
    windowed = [i for i, gspec in enumerate(runner.cache.groups) if gspec.window is not None]
    assert [runner.cache.groups[i].window for i in windowed] == [50]
    most = 0
    for i in range(0, 200, 10):
        runner.step([StepEntry("r", toks[i:i + 10], [])])
        held = sum(1 for pg in runner.cache.requests["r"].tables[windowed[0]] if pg >= 0)
        most = max(most, held)
    assert most <= (50 + 10) // page + 2
    runner.free_request("r")
    runner.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(folders, dtype):
    from qwen_engine_amd import EngineConfig, SamplingParams, generate
    cfg, _, page = TINY["B"]
    cfg_, w_ = S.read_folder(folders["B"])
    prompts = list(_requests(cfg["vocab"], (19, 3, 44), seed=12).values())
    res = generate(folders["B"], prompts, SamplingParams(max_new_tokens=12, ignore_eos=True),
                   EngineConfig(dtype=dtype, block_size=page, max_num_seqs=2, max_model_len=64, max_step_tokens=32,
                                prefill_chunk=8, debug_poison=True))
    off = 0
    for prompt, r in zip(prompts, res):
        assert r.finish_reason == "length" and len(r.token_ids) == 12
        logits = S.forward(cfg_, w_, prompt + r.token_ids[:-1]).float()
        for i, tok in enumerate(r.token_ids):
            row = logits[len(prompt) - 1 + i]
            if dtype == "float32":
                assert tok == int(row.argmax()), f"token {i} of a prompt of {len(prompt)}"
            else:
                off += not float(row.max() - row[tok]) <= 3e-2 * float(row.abs().max())
    # (in bfloat16 a router that picks one expert of four may pick another on a close call: few tokens may differ)
    assert off <= 3, f"{off} of 36 tokens are not the plain model's choice for the engine's own sequence"


def test_recorded_decode_steps_give_the_logits_of_steps_run_as_they_come(folders):
    """The same tokens through a runner that records its steps and one that runs them as they come.  (A recorded prompt
    portion is filled up to a round length, so its products run on other kernels and round otherwise: the logits agree
    to rounding but for a router's close calls, not bit for bit.)"""
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    cfg, _, page = TINY["B"]
    model = load_model(folders["B"], dtype="bfloat16")
    prompts = list(_requests(cfg["vocab"], (21, 9, 30), seed=13).values())
    fed, outs = [], []
    for use_graphs in (False, True):
        runner = ModelRunner(model, page_size=page, num_pages=24, max_requests=3, use_graphs=use_graphs)
        rows = []
        for i, p in enumerate(prompts):
            runner.add_request(i)
            rows.append(runner.step([StepEntry(i, p, [len(p) - 1])]).cpu())
        steps = [torch.cat(rows)]
        for k in range(10):
            if not use_graphs:
                fed.append([int(r.argmax()) for r in steps[-1]])
            steps.append(runner.step([StepEntry(i, [fed[k][i]], [0]) for i in range(3)]).cpu())
        outs.append(torch.cat(steps))
        if use_graphs:
            assert runner.graph_steps_of["decode"] == 10
    assert not torch.isnan(outs[1]).any()
    err = (outs[0] - outs[1]).abs().amax(dim=1) / float(outs[0].abs().max())
    assert float(err.median()) < 1.5e-2 and float((err > 6e-2).float().mean()) <= 0.1, err


def test_middling_sizes_on_the_matrix_unit_kernels(tmp_path):
    """Sizes at which the bfloat16 mode runs the matrix-unit kernels inside the engine (latent attention with key
    splits and a window, the paged attention kernels under the two maps, the tiled grouped product of the experts):
    prompts of hundreds of tokens, whole and in a mixed schedule, in both element types."""
    cfg = {
        "architecture": "Safurax", "vocab": 400, "width": 256, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-5},
        "layers": [
            {"type": "latent_attention",
             "mixer": {"heads": 6, "dim": 32, "vdim": 48, "kv_rank": 104, "q_rank": 72, "scale": 0.15},
             "mlp": {"kind": "moe", "expert": {"ff": 64}, "router": {"experts": 12, "top": 4}, "shared": {"ff": 128}}},
            {"type": "latent_attention_2",
             "mixer": {"heads": 20, "dim": 16, "rot_dim": 24, "vdim": 24, "kv_rank": 200, "scale": 0.12,
                       "rot": {"base": 10000.0, "dims": 24}, "mask": {"size": 150}},
             "mlp": {"kind": "dense", "ff": 384}},
            {"type": "attention",
             "mixer": {"heads": 6, "kv_heads": 2, "dim": 64, "vdim": 128, "diff": 0.4, "scale": 0.125,
                       "rot": {"base": 10000.0, "dims": 32, "scaling": {"factor": 2.0}}},
             "mlp": {"kind": "dense", "ff": 384}},
            {"type": "latent_attention_2",
             "mixer": {"heads": 8, "dim": 32, "rot_dim": 24, "vdim": 32, "kv_rank": 200, "scale": 0.12, "kv_from": 1,
                       "rot": {"base": 10000.0, "dims": 24}, "mask": {"size": 100}},
             "mlp": {"kind": "moe", "expert": {"ff": 96}, "router": {"experts": 5, "top": 2}, "shared": {"ff": 32}}},
        ],
    }
    folder = write_folder(str(tmp_path / "model"), cfg, random_tensors(cfg, 41))
    reqs = _requests(cfg["vocab"], (420, 300, 37, 260), seed=14)
    ref = _reference(folder, reqs)
    for dtype in ("float32", "bfloat16"):
        for cut in ("whole", "mixed"):
            trace = CUTS[cut](reqs)
            out = str(tmp_path / f"{dtype}_{cut}")
            traces.run_in_process(trace, folder, dtype, out, 16)
            got = traces.collect(trace, out, cfg["vocab"])
            if dtype == "float32":
                bad, worst = traces.first_mismatch(got, ref, 3e-4)
                assert bad is None, f"{cut}: first wrong logits at (request, position, relative error) {bad}"
            else:
                _assert_close_but_for_close_calls(got, ref, f"{dtype} {cut}")


@pytest.mark.parametrize("seed", [3, 4, 5, 11, 24, 27])
def test_configurations_drawn_at_random(tmp_path, seed):
    """Layer orders, head counts, sizes, windows and constants that no other test names, in float32 against the plain
    model, whole and in a mixed schedule."""
    cfg = random_config(seed)
    folder = write_folder(str(tmp_path / "model"), cfg, random_tensors(cfg, seed))
    reqs = _requests(cfg["vocab"], (330, 37, 150, 2, 90), seed=seed)
    ref = _reference(folder, reqs)
    for cut in ("whole", "mixed"):
        trace = CUTS[cut](reqs)
        out = str(tmp_path / cut)
        traces.run_in_process(trace, folder, "float32", out, 16)
        bad, worst = traces.first_mismatch(traces.collect(trace, out, cfg["vocab"]), ref, 3e-4)
        assert bad is None, f"{cut}: first wrong logits at (request, position, relative error) {bad}"


def test_the_command_line_with_random_weights(tmp_path, capsys):
    """main.py writes random weights for a Safurax config.json and generates from token ids."""
    import main as cli
    cfg, _, page = TINY["C"]
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(cfg))
    folder = str(tmp_path / "model")
    rc = cli.main(["--model-name-or-path", folder, "--random-weights", str(cfg_path), "--seed", "3", "--prompt-ids", "5,17,3",
                   "--prompt-ids", "9,9,100,41", "--max-new-tokens", "6", "--block-size", "16", "--max-model-len", "64",
                   "--ignore-eos", "--stats"])
    assert rc == 0
    out = capsys.readouterr().out
    assert out.count("Prompt:") == 2 and "5 17 3" in out
    stats = json.loads(out.strip().splitlines()[-1])
    assert stats["graph_steps_decode"] >= 4                 # single new tokens were replayed from recorded steps
    cfg_, w_ = S.read_folder(folder)
    assert set(w_) == set(random_tensors(cfg, 0))           # every tensor of the design, by its name
