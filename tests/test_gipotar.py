"""The Gipotar decoder in the engine against the plain implementation (``plain_gipotar.py``):
whole prompts, token-by-token decoding, portions down to two tokens, batches of unequal
requests with pages and state slots used again, long decoding, a far key made to stand out at
page borders, the first tokens of a sequence, and greedy generation through the engine's
scheduler.  Every case runs on the GPU (``-m gpu``, float32 and bfloat16) and, with the
kernels replaced by the slow torch double, on the CPU, where it tests the host logic: state
slots, input tails, the step layout."""
import copy
import json
import os

import pytest
import torch

import gipotar_models as gm
import plain_gipotar as plain
import traces
from rust_llm_inference_server_amd.config import ConfigError, EngineConfig
from rust_llm_inference_server_amd.sampling import SamplingParams

BACKENDS = ["double", pytest.param("gpu", marks=pytest.mark.gpu)]


@pytest.fixture(params=BACKENDS)
def backend(request):
    if request.param == "double":
        import cpu_ops
        cpu_ops.install(request.getfixturevalue("monkeypatch"))
        return torch.device("cpu")
    return torch.device("cuda", 0)


@pytest.fixture(params=["float32", pytest.param("bfloat16", marks=pytest.mark.gpu)])
def dtype(request, backend):
    if request.param == "bfloat16" and backend.type != "cuda":
        pytest.skip("bfloat16 runs on the GPU only")
    return request.param


_CACHE = {}


def model_case(name, dtype, tmp_path_factory, weights=None, tag=""):
    """(folder, config, the stored numbers in float64) of a configuration; made once."""
    key = (name, dtype, tag)
    if key not in _CACHE:
        cfg = gm.CONFIGS[name]
        w = weights if weights is not None else gm.make_weights(cfg, seed=len(name) + 7)
        store = torch.float32 if dtype == "float32" else torch.bfloat16
        folder = gm.write_folder(tmp_path_factory.mktemp(f"gipotar_{name}_{dtype}{tag}"), cfg, w,
                                 store, drop_rank=True)
        _CACHE[key] = (folder, cfg, gm.as_stored(w, store))
    return _CACHE[key]


def runner_for(folder, device, dtype, num_pages=64, page_size=16, max_num_seqs=4,
               max_positions=512, use_graphs=True):
    from rust_llm_inference_server_amd.engine import ModelRunner, load_model
    model = load_model(folder, dtype, max_positions, device)
    return ModelRunner(model, num_pages=num_pages, page_size=page_size,
                       max_num_seqs=max_num_seqs, use_graphs=use_graphs)


def check_trace(runner, steps, reqs, cfg, stored, dtype):
    """Replay ``steps`` and hold every wanted row against the plain logits of its request."""
    outputs = traces.replay_in_process(runner, steps)
    got = traces.collect(steps, outputs, cfg["vocab"])
    errors = []
    for rid, tokens in reqs.items():
        want = plain.forward(cfg, stored, tokens)
        assert sorted(got[rid]) == list(range(len(tokens)))
        errors += [gm.row_error(row, want[pos]) for pos, row in got[rid].items()]
    gm.judge(errors, dtype)


# ----------------------------------------------------------------------- configuration
def test_config_round_trip_and_rank_from_the_tensors(tmp_path):
    from rust_llm_inference_server_amd.registry import architecture_of
    arch = architecture_of(gm.CONFIG_A)
    assert arch.name == "Gipotar"
    cfg = arch.parse_config(gm.CONFIG_A)
    assert arch.config_to_dict(cfg) == gm.CONFIG_A
    bare = copy.deepcopy(gm.CONFIG_A)
    for layer in bare["layers"]:
        if layer["type"] == "parallel":
            del layer["mixer"]["right"]["rank"]
    cfg = arch.parse_config(bare)
    with pytest.raises(ConfigError, match=r"layers\[1\].*rank"):
        arch.build_spec(cfg)
    full = arch.complete_config(cfg, {"l1.mix.right.w1": (8, 48), "l2.mix.right.w1": (5, 48)})
    assert arch.config_to_dict(full) == gm.CONFIG_A
    names = {t.name: tuple(t.shape) for t in arch.build_spec(full).tensor_specs()}
    assert names["l0.mix.q.conv"] == (32, 3) and names["l0.mix.v"] == (96, 48)
    assert names["l1.mix.left.v"] == (64, 48) and names["l1.mix.left.o"] == (48, 128)
    assert names["l1.mix.right.u"] == (3, 16) and names["l2.mix.right.w2"] == (48, 5)
    assert "l1.norm2" not in names and "l1.mlp.gate" not in names and "l0.norm2" in names
    assert names["final.norm"] == (48,) and names["head"] == (97, 48) and names["embed"] == (97, 48)


@pytest.mark.parametrize("edit, message", [
    (lambda c: c["layers"][0].update(type="conv"), r"layers\[0\].*type 'conv'"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), r"layers\[0\] mixer.*'heads' 3"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=7), r"rot: 'dims' 7"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=18), r"rot: 'dims' 18"),
    (lambda c: c["layers"][1]["mixer"].pop("left_scale"), r"'left_scale' is missing"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), r"kind 'routed'"),
    (lambda c: c["layers"][0]["mlp"].update(limit=0.0), r"'limit' must be positive"),
    (lambda c: c.pop("residual_mult"), r"'residual_mult' is missing"),
    (lambda c: c.update(logit_softcap=0), r"'logit_softcap' must be positive"),
    (lambda c: c.update(layers=[]), r"'layers' must be a non-empty list"),
    (lambda c: c["norm"].pop("eps"), r"norm: required key 'eps'"),
])
def test_config_errors_name_the_key(edit, message):
    from rust_llm_inference_server_amd.config.gipotar import GipotarConfig
    cfg = copy.deepcopy(gm.CONFIG_A)
    edit(cfg)
    with pytest.raises(ConfigError, match=message):
        GipotarConfig.from_dict(cfg)


def test_the_plain_implementation_does_not_look_ahead():
    """The oracle's own sanity: logits of a prefix are the prefix of the logits, and every
    mechanism moves them (a constant zeroed or a layer left out changes the result)."""
    cfg = gm.CONFIG_A
    w = gm.as_stored(gm.make_weights(cfg, 3), torch.float32)
    tokens = gm.prompts(cfg["vocab"], [14], 5)[0]
    full = plain.forward(cfg, w, tokens)
    assert torch.allclose(plain.forward(cfg, w, tokens[:9]), full[:9], atol=1e-10)
    for edit in (lambda c: c.update(residual_mult=0.5), lambda c: c["embedding"].update(scale=1.0),
                 lambda c: c["layers"][1]["mixer"].update(right_scale=0.0),
                 lambda c: c["layers"][1]["mixer"].update(left_scale=0.0),
                 lambda c: c["layers"][0]["mlp"].update(limit=0.1),
                 lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=4),
                 lambda c: c.update(logit_softcap=2.0), lambda c: c["layers"].pop()):
        other = copy.deepcopy(cfg)
        edit(other)
        assert gm.row_error(plain.forward(other, w, tokens)[-1], full[-1]) > 1e-3


# --------------------------------------------------------------------- the step function
@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_whole_prompts_and_first_tokens(backend, dtype, name, tmp_path_factory):
    folder, cfg, stored = model_case(name, dtype, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [1, 2, 3, 19, 70], seed=11)
    steps, _ = traces.trace_whole(reqs)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


@pytest.mark.parametrize("name", ["a", "b"])
def test_decoding_token_by_token_equals_the_prompt_pass(backend, dtype, name, tmp_path_factory):
    """One request decoded from its first token on, one after a prompt; single tokens go
    through captured steps on the GPU."""
    folder, cfg, stored = model_case(name, dtype, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [45, 60], seed=12)
    ids = list(reqs)
    steps, _ = traces.trace_tail({ids[0]: reqs[ids[0]]}, tail=44)
    more, _ = traces.trace_tail({ids[1]: reqs[ids[1]]}, tail=33)
    for s in more:
        s["step"] += len(steps)
    check_trace(runner_for(folder, backend, dtype), steps + more, reqs, cfg, stored, dtype)


@pytest.mark.parametrize("name", ["a", "b"])
def test_portions_of_any_size(backend, dtype, name, tmp_path_factory):
    """Portions of 7, 2, 16, 3, 24, 2, 33, ... tokens: tails shorter than the taps, portions
    that end inside a page."""
    folder, cfg, stored = model_case(name, dtype, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [90, 37], seed=13)
    steps, _ = traces.trace_portions(reqs)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_mixed_batches_reuse_pages_and_state_slots(backend, dtype, name, tmp_path_factory):
    """Seven unequal requests through three state slots and a pool that holds three of them:
    portions beside single tokens, requests left out of steps, slots and pages of finished
    requests taken by later ones with their old contents still there."""
    folder, cfg, stored = model_case(name, dtype, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [50, 9, 75, 33, 2, 64, 21], seed=14)
    steps, peak = traces.trace_mixed(reqs, live=3, seed=5)
    runner = runner_for(folder, backend, dtype, num_pages=-(-peak // 16), max_num_seqs=3)
    check_trace(runner, steps, reqs, cfg, stored, dtype)
    assert runner.cache.num_free_pages() == -(-peak // 16)


def test_a_request_alone_equals_itself_in_a_batch(backend, dtype, tmp_path_factory):
    """The rows of a request do not depend on what else the step holds (beyond rounding)."""
    folder, cfg, stored = model_case("a", dtype, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [40, 23, 31], seed=15)
    alone = {}
    for rid, tokens in reqs.items():
        steps, _ = traces.trace_portions({rid: tokens})
        out = traces.replay_in_process(runner_for(folder, backend, dtype), steps)
        alone[rid] = traces.collect(steps, out, cfg["vocab"])[rid]
    steps, _ = traces.trace_mixed(reqs, live=3, seed=2)
    out = traces.replay_in_process(runner_for(folder, backend, dtype), steps)
    together = traces.collect(steps, out, cfg["vocab"])
    gm.judge([gm.row_error(row, alone[rid][pos]) for rid in reqs
              for pos, row in together[rid].items()], dtype)


@pytest.mark.parametrize("live", [20, 40])
def test_decode_steps_of_many_requests(backend, dtype, live, tmp_path_factory):
    """Twenty and forty requests decoding together (the products' kernels for 17 to 32 and for
    33 to 64 rows, their float32 results from partial sums, captured steps of those sizes), each
    row against its request's plain logits; prompts of unequal length arrive in two steps."""
    from rust_llm_inference_server_amd.engine import StepEntry
    folder, cfg, stored = model_case("a", dtype, tmp_path_factory)
    if backend.type == "cpu" and live > 20:
        pytest.skip("the double has one kernel for every row count")
    prompts = gm.prompts(cfg["vocab"], [3 + (7 * i) % 23 for i in range(live)], seed=23)
    new = 5
    tails = gm.prompts(cfg["vocab"], [new] * live, seed=24)
    runner = runner_for(folder, backend, dtype, num_pages=4 * live, max_num_seqs=live)
    errors = []
    want = [plain.forward(cfg, stored, p + t) for p, t in zip(prompts, tails)]
    for lo, hi in ((0, live // 2), (live // 2, live)):
        for i in range(lo, hi):
            runner.reserve(i, len(prompts[i]) + new)
        out = runner.step([StepEntry(i, prompts[i], [len(prompts[i]) - 1]) for i in range(lo, hi)])
        errors += [gm.row_error(out[j].cpu(), want[i][len(prompts[i]) - 1])
                   for j, i in enumerate(range(lo, hi))]
    for k in range(new):
        out = runner.step([StepEntry(i, [tails[i][k]], [0]) for i in range(live)])
        errors += [gm.row_error(out[i].cpu(), want[i][len(prompts[i]) + k]) for i in range(live)]
    gm.judge(errors, dtype)


def test_long_decoding(backend, dtype, tmp_path_factory):
    """Hundreds of single-token steps after a short prompt: the state is carried, never
    rebuilt, and what the first tokens wrote still counts at the end (slow decays)."""
    folder, cfg, stored = model_case("b", dtype, tmp_path_factory)
    n = 150 if backend.type == "cpu" else 330
    reqs = traces.random_requests(cfg["vocab"], [n], seed=16)
    steps, _ = traces.trace_tail(reqs, tail=n - 6)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


@pytest.mark.parametrize("far", [0, 15, 16, 17, 63, 64])
def test_a_far_key_that_stands_out(backend, dtype, far, tmp_path_factory):
    """One query and one key of the first layer's attention are scaled so that the token at
    ``far`` (a page's first or last position among them) takes nearly all the weight of a
    query near the end, in a prompt's portion and decoded alone.  Were that key lost or read
    from a wrong page, the first layer's attention would return another token's value."""
    cfg = gm.CONFIG_B
    w = gm.make_weights(cfg, seed=21)
    key_token, query_token = 5, 9
    left = cfg["layers"][0]["mixer"]["left"]
    d, rot = left["dim"], left["rot"]["dims"]
    probe = torch.zeros(d)
    probe[rot:] = 1.0                                   # dims that the rotation leaves alone
    for name, token in (("l0.mix.left.k", key_token), ("l0.mix.left.q", query_token)):
        direction = w["embed"][token] / w["embed"][token].norm()
        for head in range(left["heads"] if name.endswith("q") else left["kv_heads"]):
            w[name][head * d:(head + 1) * d] += 0.25 * torch.outer(probe, direction)
    folder, _, stored = model_case("b", dtype, tmp_path_factory, weights=w, tag=f"far")
    tokens = [t if t not in (key_token, query_token) else 1
              for t in gm.prompts(cfg["vocab"], [100], seed=22)[0]]
    tokens[far] = key_token
    tokens[90] = tokens[97] = query_token               # one in the prompt's part, one decoded
    # the construction works: in every head of the first layer the far key takes most of the
    # softmax weight of the query at 90 (one score stands out among ninety)
    p0 = left
    x = stored["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    h = plain.offset_norm(x, stored["l0.norm1"], cfg["norm"]["eps"])
    pos = torch.arange(len(tokens))
    q = plain.rotate((h @ stored["l0.mix.left.q"].T).reshape(-1, p0["heads"], d), pos, rot,
                     p0["rot"]["base"])
    k = plain.rotate((h @ stored["l0.mix.left.k"].T).reshape(-1, p0["kv_heads"], d), pos, rot,
                     p0["rot"]["base"])
    for head in range(p0["heads"]):
        scores = (k[:91, head // (p0["heads"] // p0["kv_heads"])] @ q[90, head]) * p0["scale"]
        assert float(torch.softmax(scores, 0)[far]) > 0.8
    reqs = {"r": tokens}
    steps, _ = traces.trace_tail(reqs, tail=6)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


def test_a_state_slot_is_cleared_for_its_next_request(backend, dtype, tmp_path_factory):
    """One slot, two requests one after the other: the second starts from zeros, not from
    what the first left (which, with these decays, would move its logits far)."""
    folder, cfg, stored = model_case("a", dtype, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [30, 12], seed=17)
    steps, _ = traces.trace_whole(reqs)
    runner = runner_for(folder, backend, dtype, max_num_seqs=1)
    check_trace(runner, steps, reqs, cfg, stored, dtype)


# -------------------------------------------------------------------- engine and scheduler
def test_greedy_generation_through_the_engine(backend, dtype, tmp_path_factory):
    """Five requests through three seats with a token budget that cuts the prompts: every
    generated token is the plain implementation's pick, up to a near-tie of its logits."""
    from rust_llm_inference_server_amd.engine import Engine, load_model
    folder, cfg, stored = model_case("a", dtype, tmp_path_factory)
    model = load_model(folder, dtype, 256, backend)
    engine = Engine(model, EngineConfig(max_num_seqs=3, max_batched_tokens=16, num_pages=48,
                                        block_size=8, max_seq_len=256, watermark_pages=1))
    prompts = gm.prompts(cfg["vocab"], [5, 21, 1, 34, 12], seed=18)
    outs = engine.generate(prompts, SamplingParams.greedy(7))
    margin = 1e-3 if dtype == "float32" else 0.5
    for p, o in zip(prompts, outs):
        assert o.finish_reason == "length" and len(o.token_ids) == 7
        tokens = list(p)
        for got in o.token_ids:
            last = plain.forward(cfg, stored, tokens)[-1]
            best = int(torch.argmax(last))
            if got != best:
                assert float(last[best] - last[got]) < margin
            tokens.append(got)
    assert engine.runner.cache.num_free_pages() == 48
    engine.runner.cache.check_invariants()


def test_preempted_requests_recompute_their_state(backend, tmp_path_factory):
    """So few pages that running requests are parked and later recomputed from their first
    token: their state slots are cleared and rebuilt, and the tokens are those of a roomy run."""
    from rust_llm_inference_server_amd.engine import Engine, load_model
    folder, cfg, stored = model_case("b", "float32", tmp_path_factory)
    model = load_model(folder, "float32", 128, backend)
    prompts = gm.prompts(cfg["vocab"], [9] * 6, seed=25)
    sp = SamplingParams.greedy(20)
    runs = []
    for pages in (64, 12):
        engine = Engine(model, EngineConfig(max_num_seqs=6, max_batched_tokens=64, num_pages=pages,
                                            block_size=8, max_seq_len=128, watermark_pages=0))
        runs.append([o.token_ids for o in engine.generate(prompts, sp)])
        assert (engine.stats().preemptions > 0) == (pages == 12)
        assert engine.runner.cache.num_free_pages() == pages
        engine.runner.cache.check_invariants()
    for roomy, tight, p in zip(runs[0], runs[1], prompts):
        if roomy != tight:                      # only at a near-tie of the plain logits
            at = next(i for i, (a, b) in enumerate(zip(roomy, tight)) if a != b)
            last = plain.forward(cfg, stored, list(p) + roomy[:at])[-1]
            assert abs(float(last[roomy[at]] - last[tight[at]])) < 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_the_replay_program_runs_the_model(dtype_name, tmp_path_factory, tmp_path):
    folder, cfg, stored = model_case("a", dtype_name, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [40, 9, 26, 3, 30], seed=19)
    steps, peak = traces.trace_mixed(reqs, live=4, seed=3)
    out = traces.replay_program(folder, dtype_name, steps, peak, str(tmp_path / "out"),
                                cfg["vocab"])
    got = traces.collect(steps, out, cfg["vocab"])
    errors = []
    for rid, tokens in reqs.items():
        want = plain.forward(cfg, stored, tokens)
        errors += [gm.row_error(row, want[pos]) for pos, row in got[rid].items()]
    gm.judge(errors, dtype_name)


@pytest.mark.gpu
def test_the_command_line_generates_and_scores(tmp_path_factory, tmp_path, capsys):
    """``rlis generate`` picks the design by config.json and prints the plain implementation's
    greedy tokens; ``rlis perplexity`` scores a token file through the same step function."""
    from rust_llm_inference_server_amd import cli
    folder, cfg, stored = model_case("a", "float32", tmp_path_factory)
    prompt = gm.prompts(cfg["vocab"], [11], seed=20)[0]
    rc = cli.main(["generate", "--model", folder, "--dtype", "f32", "--max-seq-len", "128",
                   "--num-pages", "32", "--block-size", "8", "--max-num-seqs", "2",
                   "--max-tokens", "5", "--prompt-ids", ",".join(map(str, prompt))])
    out = capsys.readouterr()
    assert rc == 0
    want, margins = plain.greedy(cfg, stored, prompt, 5)
    got = [int(t) for t in out.out.split()]
    for g, w, m in zip(got, want, margins):
        if g != w:
            assert m < 1e-3
            break
    assert len(got) == 5 and "output 5 tok (length)" in out.err
    ids = tmp_path / "ids.txt"
    tokens = gm.prompts(cfg["vocab"], [96], seed=21)[0]
    ids.write_text(" ".join(map(str, tokens)))
    rc = cli.main(["perplexity", "--model", folder, "--dtype", "f32", "--max-seq-len", "128",
                   "--ids-file", str(ids), "--ctx", "32"])
    out = capsys.readouterr()
    assert rc == 0 and json.loads(out.out.strip().splitlines()[-1])["ppl"] > 1.0
