"""The Nufavik decoder through the engine (model registry, loader, cache manager, step function, scheduler,
entry point) against the plain implementation, in every cutting of the requests."""
import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import nufavik_plain as N
import traces
from nufavik_tiny import NA, TINY, make_folder, random_tensors, write_folder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("nufavik")
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
    cfg, _, page = TINY[which]
    reqs = _requests(cfg["vocab"], (70, 33, 121, 58, 2, 95), seed=7)
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
        _assert_close_but_for_close_calls(got[cut], ref, f"{cut} against the plain model")
    whole = {rid: torch.stack([torch.from_numpy(got["whole"][rid][p]) for p in range(len(t))]) for rid, t in reqs.items()}
    for cut in ("mixed", "portions", "tail"):
        _assert_close_but_for_close_calls(got[cut], whole, f"{cut} against whole prompts")


def test_long_decoding_over_many_pages_past_every_window(folders, tmp_path):
    """Five tokens of prompt, then one at a time: every window passes over decoded tokens, pages behind the windows go
    back while the pages of the kept first keys stay."""
    cfg, _, page = TINY["A"]
    reqs = _requests(cfg["vocab"], (230,), seed=9)
    ref = _reference(folders["A"], reqs)
    trace = traces.tail_decoded(reqs, tail=225)
    out = str(tmp_path / "out")
    traces.run_in_process(trace, folders["A"], "float32", out, page)
    bad, worst = traces.first_mismatch(traces.collect(trace, out, cfg["vocab"]), ref, 2e-4)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"


def _one_layer(size, keep, seed=41):
    """One layer: what its last query sees or does not see at the window's edge and among the kept first keys
    decides its logits, since nothing else carries a token's identity forward."""
    cfg = dict(NA, layers=[dict(NA["layers"][0], mixer=dict(NA["layers"][0]["mixer"], mask={"size": size, "keep_first": keep}))])
    return cfg, random_tensors(cfg, seed, torch.float32)


@pytest.mark.parametrize("size,keep,page", [(16, 0, 8), (17, 4, 8), (24, 9, 8), (5, 1, 4), (33, 16, 16), (40, 33, 16)])
def test_keys_just_inside_and_just_outside_the_window_and_the_kept_first_keys(tmp_path, size, keep, page):
    """Changing one token changes the logits of later positions exactly where the plain model says: the token
    keep - 1 is seen from everywhere, the token keep only inside the window; position p sees the key p - size + 1 and
    not the key p - size.  Prompts and single decoded tokens alike, with the edges falling on and beside page borders."""
    cfg, w = _one_layer(size, keep)
    folder = write_folder(str(tmp_path / "model"), cfg, w)
    cfg_, w_ = N.read_folder(folder)
    g = torch.Generator().manual_seed(size + keep)
    base = torch.randint(0, cfg["vocab"], (3 * size + 40,), generator=g).tolist()
    n = len(base)
    reqs, ref = {"base": base}, {}
    # (a token reaches the keys of its own position and, through the convolution, of the taps - 1 positions behind it)
    taps = cfg["layers"][0]["mixer"]["conv"]
    for name, p in (("kept", keep - 1), ("next", keep), ("edge", n - size - (taps - 1)), ("out", n - size - taps)):
        if p < 0:
            continue
        other = list(base)
        other[p] = (base[p] + 1) % cfg["vocab"]
        reqs[name] = other
    for rid, toks in reqs.items():
        ref[rid] = N.forward(cfg_, w_, toks).float()
    last = ref["base"][-1]
    scale = float(last.abs().max())
    if keep > 0:
        assert float((ref["kept"][-1] - last).abs().max()) > 5e-5 * scale          # a kept key is seen from the end
    assert float((ref["next"][-1] - last).abs().max()) < 1e-6 * scale              # the one behind them is not
    assert float((ref["edge"][-1] - last).abs().max()) > 5e-5 * scale              # the window's oldest key is seen
    assert float((ref["out"][-1] - last).abs().max()) < 1e-6 * scale               # the one before it is not
    for cut, trace in (("whole", traces.whole(reqs)), ("tail", traces.tail_decoded(reqs, tail=size + 9)),
                       ("portions", traces.portions(reqs))):
        out = str(tmp_path / cut)
        traces.run_in_process(trace, folder, "float32", out, page)
        got = traces.collect(trace, out, cfg["vocab"])
        bad, worst = traces.first_mismatch(got, ref, 2e-5)       # (well below what one key more or less changes)
        assert bad is None, f"{cut}: first wrong logits at (request, position, relative error) {bad}"


def test_slots_and_pages_that_come_back_start_clean(folders):
    """A request that takes over the state slot and the pages of one that ended computes what it computes alone: the
    convolutions' state starts from zeros, no old key is seen."""
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


def test_a_window_gives_pages_back_and_keeps_those_of_the_first_keys(folders):
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    cfg, _, page = TINY["A"]                                # groups: windows 24 (keeps 3), 7, 37 (keeps 20), 9 (keeps 12)
    runner = ModelRunner(load_model(folders["A"], dtype="float32"), page_size=page, num_pages=40, max_requests=1)
    toks = _requests(cfg["vocab"], (150,), seed=12)["q0"]
    runner.add_request("a")
    runner.step([StepEntry("a", toks[:100], [])])
    for t in toks[100:]:
        runner.step([StepEntry("a", [t], [0])])
    runner.cache.check_invariants()
    held = {}
    for g, grp in enumerate(runner.cache.groups):
        table = runner.cache.block_table("a", g)
        held[(grp.window, grp.keep_first)] = [i for i, pg in enumerate(table) if pg >= 0]
    assert held[(7, 0)] == [18]                             # the next query, at 150, sees 144 .. 150
    assert held[(24, 3)] == [0, 15, 16, 17, 18]
    assert held[(37, 20)] == [0, 1, 2, 14, 15, 16, 17, 18]
    assert held[(9, 12)] == [0, 1, 17, 18]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(folders, dtype):
    from qwen_engine_amd import EngineConfig, SamplingParams, generate
    cfg, _, page = TINY["B"]
    cfg_, w_ = N.read_folder(folders["B"])
    prompts = list(_requests(cfg["vocab"], (19, 3, 44), seed=12).values())
    res = generate(folders["B"], prompts, SamplingParams(max_new_tokens=12, ignore_eos=True),
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
                assert float(row.max() - row[tok]) <= 3e-2 * float(row.abs().max()), f"token {i} of a prompt of {len(prompt)}"


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
        for _ in range(10):
            last = runner.step([StepEntry(i, [last[i]], [0]) for i in range(3)], greedy=True)
            rows.append(list(last))
        outs.append(rows)
        if use_graphs:
            assert runner.graph_steps_of["decode"] == 10
    assert outs[0] == outs[1]


def test_command_line_with_random_weights(tmp_path, capsys):
    """main.py writes random weights for a Nufavik config.json and generates from token ids."""
    import json
    import main as cli
    cfg, _, page = TINY["B"]
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(cfg))
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
# for several key splits of the decode kernel, many tiles of the prefill kernel and enough (token, choice) pairs for
# the tiled grouped product; windows and kept first keys that cross several pages and tiles.
NM = {"architecture": "Nufavik", "vocab": 701, "width": 320, "embedding": {"scale": 1.3}, "norm": {"eps": 1e-5},
      "layers": [
          {"type": "attention",
           "mixer": {"heads": 6, "kv_heads": 2, "dim": 64, "vdim": 40, "conv": 5, "scale": 0.12,
                     "mask": {"size": 150, "keep_first": 40}, "rot": {"base": 20000.0, "dims": 24}},
           "mlp": {"kind": "moe", "expert": {"ff": 64}, "router": {"experts": 12, "identity": 2, "top": 3, "scale": 1.7}}},
          {"type": "attention",
           "mixer": {"heads": 4, "kv_heads": 4, "dim": 96, "vdim": 128, "conv": 4, "scale": 0.09,
                     "mask": {"size": 70, "keep_first": 3}, "rot": {"base": 3000.0, "dims": 96}},
           "mlp": {"kind": "moe", "expert": {"ff": 128}, "router": {"experts": 6, "identity": 0, "top": 2, "scale": 1.0}}},
      ]}


@pytest.fixture(scope="module")
def medium(tmp_path_factory):
    folder = write_folder(str(tmp_path_factory.mktemp("nufavik_m") / "model"), NM, random_tensors(NM, 21))
    reqs = _requests(NM["vocab"], (610, 75, 380), seed=14)
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
    got = traces.collect(trace, out, NM["vocab"])
    if cut == "mixed":
        ref = {rid: rows[:max(got[rid]) + 1] for rid, rows in ref.items()}
    if dtype == "float32":
        bad, worst = traces.first_mismatch(got, ref, 2e-4)
        assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"
    else:
        _assert_close_but_for_close_calls(got, ref, f"{cut} against the plain model")
