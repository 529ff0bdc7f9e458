"""The Zarorax decoder through the engine (model registry, loader, cache manager, step function,
scheduler, entry point) against the plain implementation, in every cutting of the requests."""
import pytest
import torch

import qwen_engine_amd  # noqa: F401
from plain import zarorax_plain as Z
import traces
from zarorax_tiny import TINY, make_folder, random_tensors, write_folder

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("zarorax")
    return {which: make_folder(tmp, which) for which in TINY}


def _requests(vocab, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return {f"q{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}


def _reference(folder, reqs):
    cfg, w = Z.read_folder(folder)
    return {rid: Z.forward(cfg, w, toks).float() for rid, toks in reqs.items()}


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
    """Relative error of the logits at every (request, position), against the largest reference logit of the request."""
    out = []
    for rid, rows in ref.items():
        scale = float(rows.abs().max())
        out += [float((torch.from_numpy(got[rid][p]) - rows[p]).abs().max()) / scale for p in range(rows.shape[0])]
    return torch.tensor(out)


def _assert_close_but_for_close_calls(got, ref, what):
    """In bfloat16 a router's close call may fall the other way, and then that token's logits (and a little of
    what follows) differ by a choice, not by rounding: the typical position agrees to rounding, few do not, and
    nothing is NaN."""
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
    for cut in ("whole", "mixed", "portions"):
        trace = CUTS[cut](reqs)
        out = str(tmp_path / cut)
        traces.run_in_process(trace, folders[which], "bfloat16", out, page)
        got[cut] = traces.collect(trace, out, cfg["vocab"])
        _assert_close_but_for_close_calls(got[cut], ref, f"{cut} against the plain model")
    whole = {rid: torch.stack([torch.from_numpy(got["whole"][rid][p]) for p in range(len(t))]) for rid, t in reqs.items()}
    for cut in ("mixed", "portions"):
        _assert_close_but_for_close_calls(got[cut], whole, f"{cut} against whole prompts")


def test_long_decoding_over_many_pages(folders, tmp_path):
    cfg, _, page = TINY["R"]
    reqs = _requests(cfg["vocab"], (340,), seed=9)
    ref = _reference(folders["R"], reqs)
    trace = traces.tail_decoded(reqs, tail=335)               # five tokens of prompt, then one at a time
    out = str(tmp_path / "out")
    traces.run_in_process(trace, folders["R"], "float32", out, page)
    bad, worst = traces.first_mismatch(traces.collect(trace, out, cfg["vocab"]), ref, 2e-4)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"


def test_a_far_token_decides_the_logits(tmp_path):
    """One layer whose queries all point at the cache row of one early token: the stream after the layer,
    and with it the logits, then depends on that token's identity hundreds of positions later.  The same
    prompt with another token at that place gives other logits at the end, by as much in the engine as in
    the plain model; a key lost at a page border, or cut off, would show here."""
    cfg, seed, page = TINY["R"]
    cfg = dict(cfg, layers=cfg["layers"][:1])
    w = random_tensors(cfg, seed, torch.float32)
    w["l0.mix.uq"] *= 4.0                                     # sharp scores: few keys carry the weight
    folder = write_folder(str(tmp_path / "model"), cfg, w)
    g = torch.Generator().manual_seed(10)
    base = torch.randint(0, cfg["vocab"], (400,), generator=g).tolist()
    cfg_, w_ = Z.read_folder(folder)
    ref_a = Z.forward(cfg_, w_, base).float()
    # the early position whose change moves the last logits most
    moved = {}
    for p in (3, 4, 15, 16, 17, 63, 64):
        other = list(base)
        other[p] = (base[p] + 1) % cfg["vocab"]
        moved[p] = (float((Z.forward(cfg_, w_, other).float()[-1] - ref_a[-1]).abs().max()), other)
    p, (delta, other) = max(moved.items(), key=lambda kv: kv[1][0])
    assert delta > 1e-3 * float(ref_a.abs().max())
    reqs = {"a": base, "b": other}
    ref = {"a": ref_a, "b": Z.forward(cfg_, w_, other).float()}
    trace = traces.tail_decoded(reqs, tail=40)
    out = str(tmp_path / "out")
    traces.run_in_process(trace, folder, "float32", out, page)
    got = traces.collect(trace, out, cfg["vocab"])
    bad, worst = traces.first_mismatch(got, ref, 1e-4)
    assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"


def test_slots_and_pages_that_come_back_start_clean(folders):
    """A request that takes over the state slot and the pages of one that ended computes what it computes
    alone: the convolution's state starts from zeros, no old cache row is seen."""
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    cfg, _, page = TINY["P"]
    reqs = _requests(cfg["vocab"], (40, 37), seed=11)
    ref = _reference(folders["P"], reqs)
    runner = ModelRunner(load_model(folders["P"], dtype="float32"), page_size=page, num_pages=6, max_requests=1,
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


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_entry_point(folders, dtype):
    from qwen_engine_amd import EngineConfig, SamplingParams, generate
    cfg, _, page = TINY["Q"]
    cfg_, w_ = Z.read_folder(folders["Q"])
    prompts = list(_requests(cfg["vocab"], (19, 3, 44), seed=12).values())
    res = generate(folders["Q"], prompts, SamplingParams(max_new_tokens=12, ignore_eos=True),
                   EngineConfig(dtype=dtype, block_size=page, max_num_seqs=2, max_model_len=64, max_step_tokens=32,
                                prefill_chunk=8, debug_poison=True))
    for prompt, r in zip(prompts, res):
        assert r.finish_reason == "length" and len(r.token_ids) == 12
        logits = Z.forward(cfg_, w_, prompt + r.token_ids[:-1]).float()
        for i, tok in enumerate(r.token_ids):
            row = logits[len(prompt) - 1 + i]
            slack = 0.0 if dtype == "float32" else 3e-2 * float(row.abs().max())
            if dtype == "float32":
                assert tok == int(row.argmax()), f"token {i} of a prompt of {len(prompt)}"
            else:
                assert float(row.max() - row[tok]) <= slack, f"token {i} of a prompt of {len(prompt)}"


def test_recorded_decode_steps_give_the_tokens_of_steps_run_as_they_come(folders):
    from qwen_engine_amd.engine import ModelRunner, StepEntry, load_model
    cfg, _, page = TINY["Q"]
    model = load_model(folders["Q"], dtype="bfloat16")
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
    """main.py writes random weights for a Zarorax config.json and generates from token ids."""
    import json
    import main as cli
    cfg, _, page = TINY["Q"]
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
    cfg_, w_ = Z.read_folder(folder)
    assert set(w_) == set(random_tensors(cfg, 0))           # every tensor of the design, by its name


# Sizes at which the bfloat16 mode runs the kernels on the matrix units inside the engine: latents that fill several
# blocks of 16, heads that do not fill a wave's 16 columns or spill into a second group, enough (token, choice) pairs in
# a long prompt for the tiled grouped product, prompts long enough for several key splits and for blocks of four tokens.
ZM = {
    "architecture": "Zarorax", "vocab": 701, "width": 320, "postln_alpha": 2.5, "norm": {"eps": 1e-5},
    "canon": {"taps": 3},
    "layers": [
        {"type": "latent_attention",
         "mixer": {"heads": 6, "dim": 40, "rot_dim": 24, "vdim": 48, "kv_rank": 104, "q_rank": 72, "scale": 0.11,
                   "rot": {"base": 20000.0, "dims": 24}},
         "mlp": {"kind": "dense", "ff": 448}},
        {"type": "latent_attention_2",
         "mixer": {"heads": 20, "dim": 24, "rot_dim": 8, "vdim": 16, "kv_rank": 200, "scale": 0.14,
                   "rot": {"base": 3000.0, "dims": 8}},
         "mlp": {"kind": "moe", "expert": {"ff": 64, "limit": 1.2},
                 "router": {"experts": 12, "top": 3, "groups": {"count": 3, "keep": 2}}}},
        {"type": "latent_attention_2",
         "mixer": {"heads": 20, "dim": 24, "rot_dim": 8, "vdim": 16, "kv_rank": 200, "scale": 0.14,
                   "rot": {"base": 3000.0, "dims": 8}},
         "mlp": {"kind": "moe", "expert": {"ff": 64, "limit": 1.2},
                 "router": {"experts": 12, "top": 3, "groups": {"count": 3, "keep": 2}}}, "weights_of": 1},
    ],
}


@pytest.fixture(scope="module")
def medium(tmp_path_factory):
    folder = write_folder(str(tmp_path_factory.mktemp("zarorax_m") / "model"), ZM, random_tensors(ZM, 21))
    reqs = _requests(ZM["vocab"], (610, 75, 380), seed=14)
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
    got = traces.collect(trace, out, ZM["vocab"])
    if cut == "mixed":
        ref = {rid: rows[:max(got[rid]) + 1] for rid, rows in ref.items()}
    if dtype == "float32":
        bad, worst = traces.first_mismatch(got, ref, 2e-4)
        assert bad is None, f"first wrong logits at (request, position, relative error) {bad}"
    else:
        _assert_close_but_for_close_calls(got, ref, f"{cut} against the plain model")
