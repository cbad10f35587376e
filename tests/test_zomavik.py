"""Zomavik through the framework against the plain implementation of tests/plain/zomavik_plain.py.

Every test runs on three backends: the engine on the CPU with the plain torch ops standing in for the kernel
library (the host side: tables, slots, cache units, batching), and the engine on the GPU in float32 and in bfloat16
(the HIP kernels).  The models are the tiny ones of zomavik_configs.py with sharpened weights; the mechanisms alone
run as the framework's own parts (the registered mixers and feed-forwards) over a cache manager and pools of their own.
"""
import copy

import pytest
import torch

import trace_tools as tt
from plain import zomavik_plain as plain
from test_bokulorn import BACKENDS, CUTS, PartRunner, close, make_engine, ops_for, rounded, tolerance
from tiny_configs import random_ids
from zomavik_configs import ZOMAVIK, random_config, write_model


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("zomavik")
    return {name: write_model(raw, seed, str(root / name)) for name, (raw, seed) in ZOMAVIK.items()}


@pytest.fixture(scope="module")
def oracle(folders):
    cache = {}

    def get(name, ids):
        key = (name, tuple(ids))
        if key not in cache:
            cfg, tensors = plain.load_folder(folders[name])
            cache[key] = plain.forward(cfg, tensors, list(ids)).to(torch.float32)
        return cache[key]
    return get


def requests_for(name, lengths=(1, 2, 3, 21, 50, 97, 64, 33)):
    vocab = ZOMAVIK[name][0]["vocab"]
    return {f"r{i}": random_ids(vocab, n, 40 + i) for i, n in enumerate(lengths)}


def check_trace(folders, oracle, name, backend, steps, reqs, **kw):
    eng = make_engine(folders[name], backend, max_tokens=tt.peak_tokens(steps), max_requests=4, **kw)
    eng.pools.poison()          # pages and state rows that no request wrote read as NaN
    got = tt.run_in_process(eng, steps)
    for rid, ids in reqs.items():
        close(got[rid], oracle(name, ids), backend, rid)
    eng.cache.check_invariants()
    assert not eng.cache.requests
    return eng


NAMES = list(ZOMAVIK)


# ------------------------------------------------------------------ whole models through the engine
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts_and_the_first_tokens(folders, oracle, name, backend):
    reqs = requests_for(name)
    check_trace(folders, oracle, name, backend, tt.whole(reqs), reqs)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", NAMES)
def test_prefill_then_token_by_token(folders, oracle, name, backend):
    # The tail of 50 passes page borders of 16 and carries the scan's state and the convolution's inputs from a prompt
    # into single tokens, in every pass of a repeated run; a request of 51 starts decoding behind its very first token.
    reqs = requests_for(name, (60, 97, 64, 51))
    check_trace(folders, oracle, name, backend, tt.decode_tail(reqs, 50), reqs)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("seed", [3, 4])
def test_portions_down_to_two_tokens(folders, oracle, name, backend, seed):
    reqs = requests_for(name, (97, 50, 64, 7))
    steps = tt.portions(reqs, seed)
    assert any(len(s["entries"][0]["tokens"]) == 2 for s in steps)
    check_trace(folders, oracle, name, backend, steps, reqs)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("seed", [6, 7])
def test_mixed_batches_with_pages_and_slots_used_again(folders, oracle, name, backend, seed):
    reqs = requests_for(name, (33, 97, 21, 64, 50, 80, 12, 45, 3, 70))
    steps = tt.mixed(reqs, seed, max_live=4, tail=14)
    assert max(len(s["entries"]) for s in steps) >= 3
    eng = check_trace(folders, oracle, name, backend, steps, reqs)
    assert eng.cache.max_requests == 4          # ten requests went through four slots


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("page_size", [16, 48])
def test_other_page_sizes_and_batches_against_each_request_alone(folders, oracle, backend, page_size):
    from tokenizer_amd.engine import StepEntry
    name = "A"
    reqs = requests_for(name, (70, 9, 31))
    eng = make_engine(folders[name], backend, num_pages=24, page_size=page_size, max_requests=3)
    eng.pools.poison()
    for rid in reqs:
        eng.add_request(rid)
    heads = {rid: len(ids) - 5 for rid, ids in reqs.items()}
    got = {rid: [] for rid in reqs}
    logits = eng.step([StepEntry(rid, ids[:heads[rid]], list(range(heads[rid]))) for rid, ids in reqs.items()]).float().cpu()
    row = 0
    for rid in reqs:
        got[rid].append(logits[row:row + heads[rid]])
        row += heads[rid]
    for k in range(5):
        logits = eng.step([StepEntry(rid, [ids[heads[rid] + k]], [0]) for rid, ids in reqs.items()]).float().cpu()
        for row, rid in enumerate(reqs):
            got[rid].append(logits[row:row + 1])
    for rid, ids in reqs.items():
        close(torch.cat(got[rid]), oracle(name, ids), backend, rid)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["A", "C"])
def test_long_decoding(folders, oracle, name, backend):
    ids = random_ids(ZOMAVIK[name][0]["vocab"], 230, 77)
    reqs = {"long": ids}
    check_trace(folders, oracle, name, backend, tt.decode_tail(reqs, tail=227), reqs)


@pytest.mark.parametrize("backend", BACKENDS)
def test_greedy_generation_through_the_entry_point_and_the_scheduler(folders, backend):
    from tokenizer_amd.engine import GenerateParams, Scheduler, SchedulerConfig, generate
    name = "A"
    cfg, tensors = plain.load_folder(folders[name])
    prompts = [random_ids(cfg["vocab"], n, 90 + n) for n in (11, 30, 4)]
    want = [plain.greedy_generate(cfg, tensors, p, 9) for p in prompts]
    eng = make_engine(folders[name], backend, num_pages=16, max_requests=4)
    eng.pools.poison()
    alone = [generate(eng, p, GenerateParams.greedy(9)).tokens for p in prompts]
    sched = Scheduler(eng, SchedulerConfig(num_blocks=16, max_batch_size=4))
    rids = [sched.add_request(p, GenerateParams.greedy(9)) for p in prompts]
    results = sched.run()
    together = [results[rid].tokens for rid in rids]
    assert alone == together
    if backend != "gpu-bfloat16":           # (bfloat16 may pick another of two near-equal logits)
        assert alone == want
    else:
        for prompt, picked in zip(prompts, alone):
            logits = plain.forward(cfg, tensors, prompt + picked)[len(prompt) - 1:-1]
            for row, token in zip(logits, picked):
                assert float(row.max() - row[token]) <= 0.2 * float(row.std())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("cut", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("name", ["C", "A", "E"])
def test_hundreds_of_tokens(folders, oracle, dtype, cut, name):
    """Prompts long enough for the prompt kernels' tiles, the sorted routed layers and a long walk of the scan."""
    reqs = requests_for(name, (300, 17, 411, 130))
    steps = {"whole": lambda: tt.whole(reqs), "tail": lambda: tt.decode_tail(reqs, 40),
             "portions": lambda: tt.portions(reqs, 11), "mixed": lambda: tt.mixed(reqs, 12, max_live=4, tail=10)}[cut]()
    check_trace(folders, oracle, name, f"gpu-{dtype}", steps, reqs)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_replay_program_on_a_model_folder(folders, oracle, tmp_path, dtype):
    name = "B"
    reqs = requests_for(name, (40, 23, 5, 64, 31))
    steps = tt.mixed(reqs, 9, max_live=4, tail=6)
    got = tt.run_program(folders[name], dtype, steps, str(tmp_path / "out"), tt.peak_tokens(steps), ZOMAVIK[name][0]["vocab"])
    for rid, ids in reqs.items():
        close(got[rid], oracle(name, ids), f"gpu-{dtype}", rid)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("seed", list(range(1, 17)))
def test_models_drawn_from_a_seed(tmp_path, backend, seed):
    """Other numbers of layers, sizes and constants, repeated runs of every shape; whole, then cut and batched."""
    raw = random_config(seed)
    folder = write_model(raw, 100 + seed, str(tmp_path / "m"), sharpen=3.0)
    cfg, tensors = plain.load_folder(folder)
    reqs = {f"r{i}": random_ids(raw["vocab"], n, seed * 10 + i) for i, n in enumerate((37, 5, 52))}
    steps = tt.mixed(reqs, seed, max_live=3, tail=5) if seed % 2 else tt.portions(reqs, seed)
    eng = make_engine(folder, backend, max_tokens=tt.peak_tokens(steps), max_requests=3)
    eng.pools.poison()
    got = tt.run_in_process(eng, steps)
    for rid, ids in reqs.items():
        close(got[rid], plain.forward(cfg, tensors, ids).float(), backend, f"seed {seed} {rid}")


# ------------------------------------------------------------------ configuration, registry, schedule
def test_every_pass_has_cache_units_of_its_own_and_starts_with_the_input():
    from tokenizer_amd.config import ZomavikConfig
    from tokenizer_amd.models.zomavik import zomavik_spec
    from tokenizer_amd.parts import cache_needs, expected_tensors
    spec = zomavik_spec(ZomavikConfig.from_dict(ZOMAVIK["A"][0]))
    assert [entry.layer for entry in spec.schedule] == [0, 1, 2, 1, 2, 3]
    assert len({entry.cache_unit() for entry in spec.schedule}) == 6          # pages and state are never shared
    assert spec.options["pass_input"]["before"] == (1, 3)
    needs = cache_needs(spec)
    assert len(needs) == 6 and needs[4] == needs[1] and needs[5] == needs[2]
    assert needs[0].kind == "full" and needs[0].state_shape == (48 * 5 + 3 * 48,) and needs[0].v_dim == 24
    names = set(expected_tensors(spec))
    assert {"loop.in", "l0.ls1", "l0.ls2", "l3.ls1", "l1.mlp.shared.sg", "l0.mix.left.sink", "l0.mix.right.A_log"} <= names
    assert "l3.ls2" not in names and "l2.mlp.shared.sg" not in names and "l3.norm2" not in names
    plain_spec = zomavik_spec(ZomavikConfig.from_dict(ZOMAVIK["B"][0]))
    assert "pass_input" not in plain_spec.options and "loop.in" not in expected_tensors(plain_spec)
    once = zomavik_spec(ZomavikConfig.from_dict(ZOMAVIK["D"][0]))
    assert once.options["pass_input"]["before"] == (0,) and not once.extra_cache_units


def test_a_config_with_a_missing_or_misfitting_key_is_refused():
    from tokenizer_amd.config import ConfigError, ZomavikConfig
    raw = ZOMAVIK["A"][0]
    ZomavikConfig.from_dict(raw)

    def broken(change):
        bad = copy.deepcopy(raw)
        change(bad)
        with pytest.raises(ConfigError):
            ZomavikConfig.from_dict(bad)
    broken(lambda c: c["layers"][0]["mixer"]["right"].pop("conv"))
    broken(lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3))
    broken(lambda c: c["layers"][0]["mixer"].pop("left_scale"))
    broken(lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7))
    broken(lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=18))
    broken(lambda c: c["layers"][2].update(type="attention"))
    broken(lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=4))
    broken(lambda c: c["layers"][1]["mlp"]["router"].update(top=5))           # two kept groups of two hold four
    broken(lambda c: c["loop"].update(stop=9))
    broken(lambda c: c["loop"].update(stop=1))
    broken(lambda c: c.update(logit_softcap=-1.0))
    broken(lambda c: c["norm"].pop("eps"))


def test_the_registry_picks_the_design_by_its_config(folders):
    from tokenizer_amd.config import get_architecture, load_config
    cfg = load_config(folders["D"])
    assert cfg.architecture == "Zomavik" and cfg.embedding_scale == 1.0 and len(cfg.layers) == 2
    assert get_architecture("Zomavik").config_class is type(cfg)


@pytest.mark.gpu
def test_the_command_line_generates_from_a_model_folder(folders):
    """Ids in, ids out through the scheduler, and with random weights from the folder's config.json alone."""
    import subprocess
    import sys
    name = "B"
    cfg, tensors = plain.load_folder(folders[name])
    prompt = random_ids(cfg["vocab"], 19, 5)
    want = plain.greedy_generate(cfg, tensors, prompt, 7)
    run = subprocess.run([sys.executable, f"{tt.ROOT}/bin/qwen-infer", "--model", folders[name], "--dtype", "fp32",
                          "--max-tokens", "7", "--token-ids", " ".join(map(str, prompt))],
                         capture_output=True, text=True, timeout=300)
    assert run.returncode == 0, run.stderr
    assert f"generated ids: {want}" in run.stderr and "stop: MaxTokens" in run.stderr
    run = subprocess.run([sys.executable, f"{tt.ROOT}/bin/qwen-infer", "--model", folders[name], "--random-weights", "3",
                          "--max-tokens", "5", "--token-ids", "1 2 3"], capture_output=True, text=True, timeout=300)
    assert run.returncode == 0 and len(run.stdout.split()) == 5, run.stderr


# ------------------------------------------------------------------ the selective scan alone
def scan_spec(width, inner, state, rank, taps):
    from tokenizer_amd.parts import MixerSpec
    return MixerSpec("selective_scan", hidden_size=width, inner_size=inner, state_dim=state, dt_rank=rank, conv_taps=taps)


def scan_tensors(gen, width, inner, state, rank, taps, dtype, size=1.0, rate=0.0, step=0.0):
    rand = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float64)
    w = {"in": rand(2 * inner, width) * size / width ** 0.5, "conv": rand(inner, taps) * 0.5, "conv.b": rand(inner) * 0.2,
         "x": rand(rank + 2 * state, inner) * size / inner ** 0.5, "dt": rand(inner, rank) * size / rank ** 0.5,
         "dt.b": rand(inner) * 0.5 + step, "A_log": rand(inner, state) * 0.5 + rate, "D": 1 + 0.3 * rand(inner),
         "o": rand(width, inner) / inner ** 0.5}
    return {name: (t.float().double() if t.dim() == 1 or name == "conv" else rounded(t, dtype)) for name, t in w.items()}


SCAN_SIZES = [(48, 48, 5, 3, 4), (40, 36, 7, 5, 2), (32, 16, 1, 1, 1), (64, 128, 16, 8, 4), (64, 100, 20, 10, 3),
              (32, 24, 40, 6, 6), (32, 8, 130, 2, 2)]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("width,inner,state,rank,taps", SCAN_SIZES)
def test_selective_scan_alone(backend, cut, width, inner, state, rank, taps):
    ops, device, dtype = ops_for(backend)
    gen = torch.Generator().manual_seed(inner * 10 + state)
    n = 120
    w = scan_tensors(gen, width, inner, state, rank, taps, dtype, size=2.0)
    h = rounded(torch.randn(n, width, generator=gen, dtype=torch.float64), dtype)
    m = {"inner": inner, "state": state, "dt_rank": rank, "conv": taps}
    want = plain.selective_scan(h, m, w)
    runner = PartRunner("selective_scan", scan_spec(width, inner, state, rank, taps), w, backend)
    got = runner.run(h, CUTS[cut](n), rider=h[:9] * 0.5)
    assert float((got - want).abs().max()) <= tolerance(dtype, 3e-5, 6e-2) * max(1.0, float(want.abs().max()))
    # The slot is given back and taken again: the next request starts from zeros, not from what the last one left.
    runner.end("main")
    runner.end("rider")
    again = runner.run(h[:30] * 0.7, [30], rid="next")
    fresh = plain.selective_scan(h[:30] * 0.7, m, w)
    assert float((again - fresh).abs().max()) <= tolerance(dtype, 3e-5, 6e-2) * max(1.0, float(fresh.abs().max()))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width,inner,state,rank,taps", [(64, 128, 16, 8, 4), (40, 36, 7, 5, 2), (32, 24, 40, 6, 3)])
def test_long_portions_run_in_chunks_side_by_side(backend, width, inner, state, rank, taps):
    """Portions of hundreds of tokens are cut into chunks whose states are carried from one to the next: a prompt of 300
    (no multiple of a chunk), a single token, a portion of 267 that starts from the state those left, then single tokens;
    a second request's portion of 150 rides in the first step, so the two entries' chunks lie side by side."""
    ops, device, dtype = ops_for(backend)
    gen = torch.Generator().manual_seed(inner + state)
    n = 600
    w = scan_tensors(gen, width, inner, state, rank, taps, dtype, size=2.0, rate=-1.0, step=-2.0)
    h = rounded(torch.randn(n, width, generator=gen, dtype=torch.float64), dtype)
    other = rounded(torch.randn(150, width, generator=gen, dtype=torch.float64), dtype)
    m = {"inner": inner, "state": state, "dt_rank": rank, "conv": taps}
    want, want_other = plain.selective_scan(h, m, w), plain.selective_scan(other, m, w)
    runner = PartRunner("selective_scan", scan_spec(width, inner, state, rank, taps), w, backend, num_pages=60)
    first = runner.step([("other", other), ("main", h[:300])])
    rest = runner.run(h[300:], [1, 267] + [1] * 32, rider=other[:5])
    got = torch.cat([first[1], rest])
    bound = tolerance(dtype, 3e-5, 6e-2)
    assert float((first[0] - want_other).abs().max()) <= bound * max(1.0, float(want_other.abs().max()))
    assert float((got - want).abs().max()) <= bound * max(1.0, float(want.abs().max()))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("cut", list(CUTS))
def test_a_write_that_is_read_two_hundred_tokens_later(backend, cut):
    """Decays of nearly one (rates and step sizes far down) keep what a token wrote: the first tokens' inputs are made
    twenty times larger than the later ones (which makes their step sizes large too), so the late rows are mostly what the state carried all the way, through
    every cut of the sequence into steps.  Without those first tokens the late rows are others."""
    ops, device, dtype = ops_for(backend)
    width, inner, state, rank, taps, n = 32, 24, 6, 4, 3, 230
    gen = torch.Generator().manual_seed(11)
    w = scan_tensors(gen, width, inner, state, rank, taps, dtype, size=2.0, rate=-3.0, step=-4.0)
    h = torch.randn(n, width, generator=gen, dtype=torch.float64) * 0.05
    h[:3] *= 20.0
    h = rounded(h, dtype)
    m = {"inner": inner, "state": state, "dt_rank": rank, "conv": taps}
    want = plain.selective_scan(h, m, w)
    quiet = plain.selective_scan(torch.cat([h[:3] * 0.01, h[3:]]), m, w)
    assert float((want[200:] - quiet[200:]).abs().max()) > 8 * float(quiet[200:].abs().max())
    runner = PartRunner("selective_scan", scan_spec(width, inner, state, rank, taps), w, backend)
    got = runner.run(h, {"prompt": [n], "portions": [37, 2, 16, 1, 1, 29, 144], "decoded": [20] + [1] * 210}[cut], rider=h[:9])
    assert float((got - want).abs().max()) <= tolerance(dtype, 3e-5, 5e-2) * float(want.abs().max())
    assert float((got[200:] - want[200:]).abs().max()) <= tolerance(dtype, 1e-4, 8e-2) * float(want[200:].abs().max())


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_convolution_keeps_its_inputs_over_steps_shorter_than_its_taps(backend):
    """Only the oldest of five taps is set: a token's input reaches the scan four tokens later, over steps of one and
    two rows, so every kept input moves forward in the state row several times before it is read."""
    ops, device, dtype = ops_for(backend)
    width, inner, state, rank, taps, n = 16, 16, 3, 2, 5, 40
    gen = torch.Generator().manual_seed(2)
    w = scan_tensors(gen, width, inner, state, rank, taps, dtype, size=2.0)
    w["conv"] = torch.zeros(inner, taps, dtype=torch.float64)
    w["conv"][:, 0] = 1.5
    h = rounded(torch.randn(n, width, generator=gen, dtype=torch.float64), dtype)
    m = {"inner": inner, "state": state, "dt_rank": rank, "conv": taps}
    want = plain.selective_scan(h, m, w)
    runner = PartRunner("selective_scan", scan_spec(width, inner, state, rank, taps), w, backend)
    got = runner.run(h, [1, 2, 1, 1, 2, 2, 1, 3, 7] + [1] * 20)
    assert float((got - want).abs().max()) <= tolerance(dtype, 3e-5, 6e-2) * max(1.0, float(want.abs().max()))


# ------------------------------------------------------------------ the attention alone
def attention_spec(width, heads, kv_heads, d, dv, dims, base, scale, softcap):
    from tokenizer_amd.models.zomavik import _attention
    raw = {"heads": heads, "kv_heads": kv_heads, "dim": d, "vdim": dv, "scale": scale, "rot": {"dims": dims, "base": base}}
    if softcap is not None:
        raw["softcap"] = softcap
    return _attention(raw, width, 1e-6, 1 << 20), raw


def attention_tensors(gen, width, heads, kv_heads, d, dv, dtype, size=1.0):
    rand = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float64)
    w = {"q": rand(heads * d, width) * size / width ** 0.5, "q.b": rand(heads * d) * 0.3,
         "k": rand(kv_heads * d, width) * size / width ** 0.5, "k.b": rand(kv_heads * d) * 0.3,
         "v": rand(kv_heads * dv, width) / width ** 0.5, "v.b": rand(kv_heads * dv) * 0.3, "sink": rand(heads) * 2.0,
         "o": rand(width, heads * dv) / (heads * dv) ** 0.5}
    return {name: (t.float().double() if t.dim() == 1 else rounded(t, dtype)) for name, t in w.items()}


def part_names(w):
    from tokenizer_amd.models.zomavik import _ATTENTION_NAMES
    return {ours: w[theirs] for ours, theirs in _ATTENTION_NAMES}


ATTENTION_SIZES = [(48, 4, 2, 16, 24, 8, 10000.0, 0.3, 20.0), (40, 3, 3, 10, 14, 6, 300.0, 0.35, 2.0),
                   (32, 1, 1, 24, 40, 2, 100.0, 0.2, 3.0), (64, 4, 1, 64, 64, 32, 500000.0, 0.125, 30.0),
                   (64, 8, 2, 32, 32, 32, 10000.0, 0.18, 4.0), (48, 6, 2, 6, 10, 0, 100.0, 0.4, None),
                   (64, 6, 1, 48, 16, 48, 10000.0, 0.144, 50.0), (64, 2, 1, 128, 128, 64, 10000.0, 0.09, 9.0),
                   (48, 6, 2, 96, 96, 96, 1000.0, 0.1, 6.0), (40, 3, 1, 80, 80, 10, 200.0, 0.11, None)]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("width,heads,kv_heads,d,dv,dims,base,scale,softcap", ATTENTION_SIZES)
def test_capped_attention_with_a_sink_alone(backend, cut, width, heads, kv_heads, d, dv, dims, base, scale, softcap):
    ops, device, dtype = ops_for(backend)
    gen = torch.Generator().manual_seed(heads * 100 + d + dv)
    n = 120
    w = attention_tensors(gen, width, heads, kv_heads, d, dv, dtype, size=4.0)
    h = rounded(torch.randn(n, width, generator=gen, dtype=torch.float64), dtype)
    spec, m = attention_spec(width, heads, kv_heads, d, dv, dims, base, scale, softcap)
    want = plain.capped_sink_attention(h, m, w)
    runner = PartRunner("gqa_attention", spec, part_names(w), backend)
    got = runner.run(h, CUTS[cut](n), rider=h[:9] * 0.5)
    assert float((got - want).abs().max()) <= tolerance(dtype, 3e-5, 6e-2) * max(1.0, float(want.abs().max()))
    if softcap is not None and softcap < 10:      # the cap does matter here: without it the rows are others
        free = plain.capped_sink_attention(h, {**m, "softcap": None}, w)
        assert float((free - want).abs().max()) > 0.05
    loud = {**w, "sink": w["sink"] + 6.0}          # and so does the sink: a larger one takes weight from every key
    assert float((plain.capped_sink_attention(h, m, loud) - want).abs().max()) > 0.05


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("d,dv", [(16, 8), (32, 32)])
def test_one_key_made_to_stand_out_far_back_and_at_page_borders(backend, cut, d, dv):
    """The mixer's input is [a query part | a key part]: the query projection reads the first half, the key projection
    the second, through the same matrix, so a query whose first half is the second half of a chosen token scores that
    token far above all others (up to the cap, which still leaves it far above).  The chosen keys are, in turn: the
    second token of the sequence (hundreds of tokens back), the keys on either side of the last page border, the key
    before the query, the query itself and the very first token.  Nothing is rotated, so the chosen key wins at any
    distance.  A key that is lost, or one too many, changes the output by all of it."""
    ops, device, dtype = ops_for(backend)
    heads, n = 2, 230
    gen = torch.Generator().manual_seed(5 + d)
    rand = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float64)
    keys = rand(n, d)
    keys = keys / keys.norm(dim=-1, keepdim=True)
    target = []
    for i in range(n):
        j = [1, i - i % 16, i - i % 16 - 1, i - 1, i, 0][i % 6]
        target.append(j if 0 <= j <= i else i)
    h = rounded(torch.cat([keys[target], keys], dim=1), dtype)
    eye, zero = torch.eye(d, dtype=torch.float64), torch.zeros(d, d, dtype=torch.float64)
    w = {"q": torch.cat([torch.cat([eye, zero], dim=1)] * heads), "q.b": torch.zeros(heads * d, dtype=torch.float64),
         "k": torch.cat([zero, eye], dim=1), "k.b": torch.zeros(d, dtype=torch.float64),
         "v": rounded(rand(dv, 2 * d), dtype), "v.b": torch.zeros(dv, dtype=torch.float64),
         "sink": torch.tensor([-2.0, 1.0], dtype=torch.float64), "o": rounded(rand(2 * d, heads * dv) / dv ** 0.5, dtype)}
    spec, m = attention_spec(2 * d, heads, 1, d, dv, 0, 100.0, 60.0, 200.0)
    want = plain.capped_sink_attention(h, m, w)
    values = (h @ w["v"].T)
    alone = torch.cat([values[target]] * heads, dim=1) @ w["o"].T     # what a softmax on the chosen key alone gives
    assert float((want - alone).abs().max()) < 1e-3 * float(want.abs().max())
    runner = PartRunner("gqa_attention", spec, part_names(w), backend)
    got = runner.run(h, {"prompt": [n], "portions": [37, 2, 16, 1, 1, 29, 144], "decoded": [160] + [1] * 70}[cut], rider=h[:9])
    assert float((got - want).abs().max()) <= tolerance(dtype, 3e-5, 3e-2) * float(want.abs().max())


def test_two_mixers_side_by_side_ask_for_pages_and_state_together():
    from tokenizer_amd.parts import MIXERS, MixerSpec
    left, _ = attention_spec(48, 4, 2, 16, 24, 8, 100.0, 0.3, 5.0)
    right = scan_spec(48, 40, 9, 6, 3)
    both = MixerSpec("side_by_side", hidden_size=48, options={"left": left, "right": right, "left_scale": 0.3, "right_scale": 2.0})
    need = MIXERS.get("side_by_side").cache_need(both)
    assert (need.kind, need.n_kv_heads, need.head_dim, need.v_dim) == ("full", 2, 16, 24)
    assert need.state_shape == (40 * 9 + 2 * 40,)
    names = set(MIXERS.get("side_by_side").tensor_specs(both))
    assert {"left.q", "left.q.b", "left.sink", "left.o", "right.in", "right.conv.b", "right.A_log"} <= names
    twice = MixerSpec("side_by_side", hidden_size=48, options={"left": right, "right": right})
    with pytest.raises(ValueError):
        MIXERS.get("side_by_side").cache_need(twice)


# ------------------------------------------------------------------ router, experts, dense layer
def run_feed_forward(kind, spec, tensors, backend, x):
    from tokenizer_amd.parts import FEED_FORWARDS, Runtime
    ops, device, dtype = ops_for(backend)
    stored = {name: t.to(torch.float32 if t.dim() == 1 else dtype).to(device).contiguous() for name, t in tensors.items()}
    part = FEED_FORWARDS.get(kind)(spec, stored, Runtime(dtype, device, ops))
    return part.forward(x.to(dtype).to(device).contiguous(), None).double().cpu()


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,count,keep", [(12, 3, 2, 1), (6, 2, 3, 2), (5, 1, 5, 5), (8, 3, None, None), (64, 6, 8, 3),
                                                     (4, 4, 1, 1), (9, 2, 9, 3)])
def test_the_router_against_a_choice_written_out_here(backend, experts, top, count, keep):
    """Softmax over all experts, a group worth its best expert, the best groups kept, the best experts inside them,
    weights over the chosen's sum; and the gate's number behind the experts' logits."""
    ops, device, dtype = ops_for(backend)
    gen = torch.Generator().manual_seed(experts * 7 + top)
    n = 70
    logits = (torch.randn(n, experts + 1, generator=gen) * 3.0).to(device).contiguous()
    chosen = torch.empty((n, top), dtype=torch.int32, device=device)
    weights = torch.empty((n, top), dtype=torch.float32, device=device)
    gate = torch.empty((n,), dtype=torch.float32, device=device)
    ops.route_scores(logits, None, experts, count or 0, keep or 0, chosen, weights, softmax=True, group_max=True, gate=gate)
    for t in range(n):
        z = logits[t, :experts].double().cpu()
        s = torch.exp(z - z.max())
        s = s / s.sum()
        allowed = list(range(experts))
        if count:
            per = experts // count
            best = sorted(range(count), key=lambda g: -max(s[g * per:(g + 1) * per]))[:keep]
            allowed = [e for e in range(experts) if e // per in best]
        picks = sorted(allowed, key=lambda e: -s[e])[:top]
        assert chosen[t].tolist() == picks
        total = sum(s[e] for e in picks)
        assert torch.allclose(weights[t].double().cpu(), torch.stack([s[e] / total for e in picks]), atol=1e-6)
    assert torch.allclose(gate.double().cpu(), torch.sigmoid(logits[:, experts].double().cpu()), atol=1e-6)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("rows", [1, 7, 150, 700])
@pytest.mark.parametrize("width,experts,top,ff,count,keep,shared", [(64, 6, 2, 24, 3, 2, 16), (40, 5, 1, 10, 5, 5, 6), (64, 8, 3, 32, 2, 1, 32),
                                                                    (48, 4, 1, 20, None, None, None)])
def test_routed_experts_with_a_gated_shared_expert(backend, rows, width, experts, top, ff, count, keep, shared):
    """Few rows run every expert, many rows (in bfloat16) the tiles sorted by expert; both against one token and expert
    at a time."""
    from tokenizer_amd.models.zomavik import _feed_forward
    ops, device, dtype = ops_for(backend)
    if backend == "cpu" and rows > 200:
        pytest.skip("the long batches are for the sorted form on the device")
    gen = torch.Generator().manual_seed(rows + experts)
    rand = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float64)
    router = {"experts": experts, "top": top}
    if count:
        router["groups"] = {"count": count, "keep": keep}
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    names = [(f"e{j}", ff) for j in range(experts)]
    if shared:
        mlp["shared"] = {"ff": shared}
        names.append(("shared", shared))
    w = {"router": rounded(rand(experts, width) * 3.0 / width ** 0.5, dtype)}
    for name, inner in names:
        w.update({f"{name}.gate": rounded(rand(inner, width) * 2 / width ** 0.5, dtype), f"{name}.up": rounded(rand(inner, width) * 2 / width ** 0.5, dtype),
                  f"{name}.down": rounded(rand(width, inner) / inner ** 0.5, dtype)})
    if shared:
        w["shared.sg"] = rounded(rand(1, width) * 2 / width ** 0.5, dtype)
    h = rounded(rand(rows, width), dtype)
    want = plain.routed_feed_forward(h, mlp, w)
    got = run_feed_forward("routed_experts", _feed_forward(mlp, width), w, backend, h)
    off = (got - want).abs().amax(dim=-1) / max(1.0, float(want.abs().max()))
    # (bfloat16 rounds the router's input, and a row whose two best scores nearly tie may then choose the other expert.)
    assert int((off > tolerance(dtype, 3e-5, 5e-2)).sum()) <= (rows // 20 if dtype == torch.bfloat16 else 0)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width,ff,rows", [(48, 40, 33), (52, 30, 5), (128, 96, 300)])
def test_the_dense_layer_without_a_gate(backend, width, ff, rows):
    from tokenizer_amd.models.zomavik import _feed_forward
    ops, device, dtype = ops_for(backend)
    gen = torch.Generator().manual_seed(ff)
    rand = lambda *shape: torch.randn(*shape, generator=gen, dtype=torch.float64)
    w = {"up": rounded(rand(ff, width) * 2 / width ** 0.5, dtype), "down": rounded(rand(width, ff) / ff ** 0.5, dtype)}
    h = rounded(rand(rows, width), dtype)
    want = plain.dense_feed_forward(h, w)
    got = run_feed_forward("plain_dense", _feed_forward({"kind": "dense", "ff": ff}, width), w, backend, h)
    assert float((got - want).abs().max()) <= tolerance(dtype, 3e-5, 5e-2) * max(1.0, float(want.abs().max()))


# ------------------------------------------------------------------ the weighted terms with their norms, the logits' cap
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("hidden", [40, 256, 1000, 2304])
@pytest.mark.parametrize("n_terms", [0, 1, 3, 4])
def test_weighted_terms_join_the_stream_under_one_or_two_norms(backend, hidden, n_terms):
    ops, device, dtype = ops_for(backend)
    gen = torch.Generator().manual_seed(hidden + n_terms)
    rows = 9
    stream = torch.randn(rows, hidden, generator=gen).to(device)
    terms, total = [], torch.zeros(rows, hidden, dtype=torch.float64)
    for k in range(n_terms):
        part = torch.randn(rows, hidden, generator=gen).to(dtype)
        scale = None if k == 1 else (1 + 0.3 * torch.randn(hidden, generator=gen))
        factor = [0.7, 0.4, 1.0, -1.5][k]
        total += factor * part.double() * (1.0 if scale is None else scale.double())
        terms.append((part.to(device), factor, None if scale is None else scale.to(device)))
    w1, w2 = (1 + 0.3 * torch.randn(hidden, generator=gen)), (1 + 0.3 * torch.randn(hidden, generator=gen))
    x = stream.double().cpu() + total
    unit = lambda eps: x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    bound = tolerance(dtype, 1e-5, 2e-2) * max(1.0, float(x.abs().max()))
    # Two norms of the same sum, stored back.
    kept = stream.clone()
    out1 = torch.empty(rows, hidden, dtype=dtype, device=device)
    out2 = torch.empty_like(out1)
    ops.add_terms_rmsnorm(kept, terms, w1.to(device), 1e-5, out1, weight2=w2.to(device), eps2=1e-3, out2=out2)
    assert float((kept.double().cpu() - x).abs().max()) <= 1e-5 * max(1.0, float(x.abs().max()))
    assert float((out1.double().cpu() - unit(1e-5) * w1.double()).abs().max()) <= bound
    assert float((out2.double().cpu() - unit(1e-3) * w2.double()).abs().max()) <= bound
    # Some rows, nothing stored; then the sum itself into the left half of wider rows.
    kept = stream.clone()
    pick = torch.tensor([7, 0, 3], dtype=torch.int32, device=device)
    some = torch.empty(3, hidden, dtype=dtype, device=device)
    ops.add_terms_rmsnorm(kept, terms, w1.to(device), 1e-5, some, pick, store_residual=False)
    assert torch.equal(kept, stream)
    assert float((some.double().cpu() - (unit(1e-5) * w1.double())[[7, 0, 3]]).abs().max()) <= bound
    wide = torch.zeros(rows, 2 * hidden, dtype=dtype, device=device)
    ops.add_terms_rmsnorm(kept, terms, None, 0.0, wide[:, :hidden], store_residual=False)
    assert float((wide[:, :hidden].double().cpu() - x).abs().max()) <= bound and float(wide[:, hidden:].abs().max()) == 0.0


@pytest.mark.parametrize("backend", BACKENDS)
def test_scaled_and_capped_logits(backend):
    ops, device, dtype = ops_for(backend)
    z = (torch.randn(5, 333, generator=torch.Generator().manual_seed(1)) * 40).to(device)
    capped = ops.scale_cap(z.clone(), 0.3, 12.0).double().cpu()
    assert torch.allclose(capped, 12.0 * torch.tanh(z.double().cpu() * 0.3 / 12.0), atol=1e-5)
    assert torch.allclose(ops.scale_cap(z.clone(), 0.7, 0.0).double().cpu(), z.double().cpu() * 0.7, atol=1e-5)
