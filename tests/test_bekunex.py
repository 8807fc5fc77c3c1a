"""The Bekunex decoder in the engine against the plain implementation (``plain_bekunex.py``):
whole prompts, token-by-token decoding, portions down to two tokens, batches of unequal
requests with pages and state slots used again, long decoding, keys made to stand out far
away, at page borders and just inside and just outside a window, the sink, the first tokens of
a sequence, and greedy generation through the engine's scheduler.  Every case runs on the GPU
(``-m gpu``, float32 and bfloat16) and, with the kernels replaced by the slow torch double, on
the CPU, where it tests the host logic: run order and shared caches, windows, state slots,
input tails, the step layout."""
import copy
import json

import pytest
import torch

import bekunex_models as bm
import plain_bekunex as plain
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


def model_case(name, dtype, tmp_path_factory, weights=None, tag="", config=None):
    """(folder, config, the stored numbers in float64) of a configuration; made once."""
    key = (name, dtype, tag)
    if key not in _CACHE:
        cfg = config if config is not None else bm.CONFIGS[name]
        w = weights if weights is not None else bm.make_weights(cfg, seed=len(name) + 3)
        store = torch.float32 if dtype == "float32" else torch.bfloat16
        folder = bm.write_folder(tmp_path_factory.mktemp(f"bekunex_{name}_{dtype}{tag}"), cfg, w,
                                 store)
        _CACHE[key] = (folder, cfg, bm.as_stored(w, store))
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
        want = plain.forward(stored, cfg, tokens)
        assert sorted(got[rid]) == list(range(len(tokens)))
        errors += [bm.row_error(row, want[pos]) for pos, row in got[rid].items()]
    bm.judge(errors, dtype)


# ----------------------------------------------------------------------- configuration
def test_config_round_trip_and_run_order():
    from rust_llm_inference_server_amd.registry import architecture_of
    for cfg in bm.CONFIGS.values():
        arch = architecture_of(cfg)
        assert arch.name == "Bekunex"
        typed = arch.parse_config(cfg)
        assert arch.config_to_dict(typed) == cfg
        spec = arch.build_spec(typed)
        for i, run in enumerate(spec.runs()):
            assert run.layer == i and run.cache_of == cfg["layers"][i]["mixer"].get("kv_from")
    # a reader's wider window is what the writer's cache keeps
    spec = bm.spec_of(bm.CONFIG_A)
    first = spec.layers[0].block.params["mixer"].params
    reader = spec.layers[3].block.params["mixer"].params
    assert first["window"] == 20 and first["cache_window"] == 33
    assert reader["window"] == 33 and reader["cache_window"] == 33 and not reader["own_latent"]
    names = {t.name for t in spec.tensor_specs()}
    assert "l0.mix.dkv" in names and "l3.mix.dkv" not in names and "l3.mix.uk" in names
    assert "l2.mlp.shared.gate" not in names and "l0.mlp.shared.gate" in names
    assert "l1.mlp.router" not in names


def _edit(path, value):
    def apply(cfg):
        node = cfg
        for key in path[:-1]:
            node = node[key]
        if value is _DROP:
            del node[path[-1]]
        else:
            node[path[-1]] = value
    return apply


_DROP = object()


@pytest.mark.parametrize("edit, message", [
    (_edit(("layers", 0, "type"), "latent_attention_3"), "type 'latent_attention_3'"),
    (_edit(("layers", 0, "mixer", "mask"), _DROP), "'mask'"),
    (_edit(("layers", 3, "mixer", "kv_from"), 2), "'kv_from' 2"),
    (_edit(("layers", 3, "mixer", "kv_from"), 3), "'kv_from' 3"),
    (_edit(("layers", 3, "mixer", "kv_rank"), 24), "'kv_rank' 24"),
    (_edit(("layers", 2, "mixer", "rot", "dims"), 7), "'dims' 7"),
    (_edit(("layers", 2, "mixer", "rot", "dims"), 10), "'dims' 10"),
    (_edit(("layers", 1, "mixer", "state"), 0), "'state'"),
    (_edit(("layers", 0, "mlp", "kind"), "dense"), "kind 'dense'"),
    (_edit(("layers", 0, "mlp", "router", "groups", "count"), 4), "4 equal groups"),
    (_edit(("layers", 0, "mlp", "router", "top"), 5), "'top' 5"),
    (_edit(("layers", 0, "mlp", "router", "groups", "keep"), 4), "'keep' 4"),
    (_edit(("logit_scale",), _DROP), "'logit_scale'"),
    (_edit(("norm", "eps"), 0.0), "'eps'"),
])
def test_config_errors_name_the_key(edit, message):
    from rust_llm_inference_server_amd.registry import architecture_of
    cfg = copy.deepcopy(bm.CONFIG_A)
    edit(cfg)
    with pytest.raises(ConfigError) as e:
        architecture_of(cfg).parse_config(cfg)
    assert message in str(e.value)


def test_the_plain_implementation_does_not_look_ahead():
    """A position's plain logits depend on the tokens up to it and on nothing behind it; and
    they do depend on a token that has left every window (through the scans' states)."""
    cfg = bm.CONFIG_A
    stored = bm.as_stored(bm.make_weights(cfg, 5), torch.float32)
    tokens = bm.prompts(cfg["vocab"], [60], seed=1)[0]
    whole = plain.forward(stored, cfg, tokens)
    part = plain.forward(stored, cfg, tokens[:41])
    assert float((whole[:41] - part).abs().max()) < 1e-9
    other = list(tokens)
    other[3] = (other[3] + 1) % cfg["vocab"]
    assert float((plain.forward(stored, cfg, other)[-1] - whole[-1]).abs().max()) > 1e-6


# --------------------------------------------------------------------- the step function
@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
def test_whole_prompts_and_first_tokens(backend, dtype, name, tmp_path_factory):
    folder, cfg, stored = model_case(name, dtype, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [1, 2, 3, 19, 70], seed=11)
    steps, _ = traces.trace_whole(reqs)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


@pytest.mark.parametrize("name", ["a", "b", "d"])
def test_decoding_token_by_token_equals_the_prompt_pass(backend, dtype, name, tmp_path_factory):
    """One request decoded from its first token on, one after a prompt, so that every window
    passes over decoded tokens; single tokens go through captured steps on the GPU."""
    folder, cfg, stored = model_case(name, dtype, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [45, 80], seed=12)
    ids = list(reqs)
    steps, _ = traces.trace_tail({ids[0]: reqs[ids[0]]}, tail=44)
    more, _ = traces.trace_tail({ids[1]: reqs[ids[1]]}, tail=45)
    for s in more:
        s["step"] += len(steps)
    check_trace(runner_for(folder, backend, dtype), steps + more, reqs, cfg, stored, dtype)


@pytest.mark.parametrize("name", ["a", "b", "d"])
def test_portions_of_any_size(backend, dtype, name, tmp_path_factory):
    """Portions of 7, 2, 16, 3, 24, 2, 33, ... tokens: tails shorter than the taps, portions
    that end inside a page and inside a window."""
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
    bm.judge([bm.row_error(row, alone[rid][pos]) for rid in reqs
              for pos, row in together[rid].items()], dtype)


@pytest.mark.parametrize("live", [20, 40])
def test_decode_steps_of_many_requests(backend, dtype, live, tmp_path_factory):
    """Twenty and forty requests decoding together (the routed units' tiles of 16 and of 64
    rows, the products' kernels for 17 to 32 and for 33 to 64 rows, captured steps of those
    sizes), each row against its request's plain logits."""
    from rust_llm_inference_server_amd.engine import StepEntry
    folder, cfg, stored = model_case("b", dtype, tmp_path_factory)
    if backend.type == "cpu" and live > 20:
        pytest.skip("the double has one kernel for every row count")
    prompts = bm.prompts(cfg["vocab"], [3 + (7 * i) % 23 for i in range(live)], seed=23)
    new = 4
    tails = bm.prompts(cfg["vocab"], [new] * live, seed=24)
    runner = runner_for(folder, backend, dtype, num_pages=4 * live, max_num_seqs=live)
    errors = []
    want = [plain.forward(stored, cfg, p + t) for p, t in zip(prompts, tails)]
    for lo, hi in ((0, live // 2), (live // 2, live)):
        for i in range(lo, hi):
            runner.reserve(i, len(prompts[i]) + new)
        out = runner.step([StepEntry(i, prompts[i], [len(prompts[i]) - 1]) for i in range(lo, hi)])
        errors += [bm.row_error(out[j].cpu(), want[i][len(prompts[i]) - 1])
                   for j, i in enumerate(range(lo, hi))]
    for k in range(new):
        out = runner.step([StepEntry(i, [tails[i][k]], [0]) for i in range(live)])
        errors += [bm.row_error(out[i].cpu(), want[i][len(prompts[i]) + k]) for i in range(live)]
    bm.judge(errors, dtype)


def test_long_decoding(backend, dtype, tmp_path_factory):
    """Hundreds of single-token steps after a short prompt: the scans' states are carried,
    never rebuilt, windows move over many pages (which are given back), and what the first
    tokens wrote still counts at the end (slow decays)."""
    folder, cfg, stored = model_case("b", dtype, tmp_path_factory)
    n = 120 if backend.type == "cpu" else 330
    reqs = traces.random_requests(cfg["vocab"], [n], seed=16)
    steps, _ = traces.trace_tail(reqs, tail=n - 6)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


def _standing_out(cfg, layer, key_token, query_token, seed, boost=6.0):
    """Weights in which, in every head of ``layer``'s attention, the key made from
    ``key_token``'s latent takes nearly all the weight of a query made from ``query_token``:
    one latent direction that only the key token's down projection fills and that every head's
    key map sends to a direction its query map answers."""
    w = bm.make_weights(cfg, seed=seed)
    m = cfg["layers"][layer]["mixer"]
    p = f"l{layer}.mix"
    H, d, R = m["heads"], m["dim"], m["kv_rank"]
    dq = d + m.get("rot_dim", 0)
    emb = w["embed"]
    # the first layer's normed input is a fixed function of the token: make the two directions
    # from it, so that they survive the norm's weight and bias
    h = plain.layer_norm(emb.double(), w[p.replace(".mix", ".norm1")].double(),
                         w[p.replace(".mix", ".norm1.b")].double(), cfg["norm"]["eps"]).float()
    hk, hq = h[key_token] / h[key_token].norm(), h[query_token] / h[query_token].norm()
    w[p + ".dkv"][0] += boost * hk              # latent channel 0 answers the key token
    for head in range(H):
        w[p + ".uk"][head * d] *= 0.0
        w[p + ".uk"][head * d, 0] = boost       # ... and becomes key dim 0 of every head
        w[p + ".q"][head * dq] += boost * hq    # which the query token's query dim 0 meets
    return w


@pytest.mark.parametrize("far", [0, 15, 16, 17, 63, 64])
def test_a_far_key_that_stands_out(backend, dtype, far, tmp_path_factory):
    """Full causal attention over cached latents: the token at ``far`` (a page's first or last
    position among them) takes most of the weight of a query near the end, in a prompt's
    portion and decoded alone.  Were its row lost or read from a wrong page, the layer would
    return another token's value."""
    cfg = copy.deepcopy(bm.CONFIG_B)
    key_token, query_token = 5, 9
    w = _standing_out(cfg, 0, key_token, query_token, seed=21)
    folder, _, stored = model_case("b", dtype, tmp_path_factory, weights=w, tag="far", config=cfg)
    tokens = [t if t not in (key_token, query_token) else 1
              for t in bm.prompts(cfg["vocab"], [100], seed=22)[0]]
    tokens[far] = key_token
    tokens[90] = tokens[97] = query_token
    # the construction works: moving the key token moves the query's logits far
    moved = list(tokens)
    moved[far] = 1
    a, b = plain.forward(stored, cfg, tokens), plain.forward(stored, cfg, moved)
    assert bm.row_error(a[90], b[90]) > 0.05 and bm.row_error(a[97], b[97]) > 0.05
    reqs = {"r": tokens}
    steps, _ = traces.trace_tail(reqs, tail=6)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


@pytest.mark.parametrize("back", [19, 20, 32, 33])
def test_keys_just_inside_and_outside_a_window(backend, dtype, back, tmp_path_factory):
    """Two layers read one cache under windows of 20 and 33 positions.  A key that stands out
    lies ``back`` positions behind the query: the last one inside or the first one outside of
    either window.  A window that is one token off, in a prompt's portion or decoded alone,
    moves the row far."""
    cfg = copy.deepcopy(bm.CONFIG_A)
    key_token, query_token = 5, 9
    w = _standing_out(cfg, 0, key_token, query_token, seed=31)
    # the reader of the same cache looks for the same latent channel
    m3 = cfg["layers"][3]["mixer"]
    for head in range(m3["heads"]):
        w["l3.mix.uk"][head * m3["dim"]] *= 0.0
        w["l3.mix.uk"][head * m3["dim"], 0] = 6.0
        w["l3.mix.q"][head * m3["dim"]] += 2.0 * w["l0.mix.q"][0] / w["l0.mix.q"][0].norm()
    folder, _, stored = model_case("a", dtype, tmp_path_factory, weights=w, tag="edge", config=cfg)
    tokens = [t if t not in (key_token, query_token) else 1
              for t in bm.prompts(cfg["vocab"], [130], seed=32)[0]]
    queries = (60, 120)                         # one in the prompt's part, one decoded
    for query in queries:
        tokens[query] = query_token
        tokens[query - back] = key_token
    # the construction works: with both windows one position off (shorter when the key is the
    # last one inside, longer when it is the first one outside) the plain logits move far
    other = copy.deepcopy(cfg)
    for i in (0, 3):
        other["layers"][i]["mixer"]["mask"]["size"] += -1 if back in (19, 32) else 1
    a, b = plain.forward(stored, cfg, tokens), plain.forward(stored, other, tokens)
    for query in queries:
        assert bm.row_error(a[query], b[query]) > 0.03
    reqs = {"r": tokens}
    steps, _ = traces.trace_tail(reqs, tail=12)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)
    steps, _ = traces.trace_portions(reqs)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


def test_the_sink_counts_once_and_unscaled(backend, dtype, tmp_path_factory):
    """Sinks far above the scores: the heads' outputs nearly vanish.  An engine that left the
    sink out, scaled it or counted it per key would be far off."""
    cfg = bm.CONFIG_D
    w = bm.make_weights(cfg, seed=41)
    for i in (1, 2, 3):
        w[f"l{i}.mix.sink"] = torch.tensor([3.0, -2.0, 5.0, 0.5][:w[f"l{i}.mix.sink"].numel()])
    folder, _, stored = model_case("d", dtype, tmp_path_factory, weights=w, tag="sink")
    without = {k: (v - 30.0 if k.endswith(".sink") else v) for k, v in stored.items()}
    reqs = traces.random_requests(cfg["vocab"], [40], seed=42)
    tokens = reqs["r0"]
    assert bm.row_error(plain.forward(stored, cfg, tokens)[-1],
                        plain.forward(without, cfg, tokens)[-1]) > 0.05
    steps, _ = traces.trace_tail(reqs, tail=5)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


def test_a_state_slot_is_cleared_for_its_next_request(backend, dtype, tmp_path_factory):
    """One slot, two requests one after the other: the second starts from zeros, not from
    what the first left (which, with these decays, would move its logits far)."""
    folder, cfg, stored = model_case("c", dtype, tmp_path_factory)
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
    prompts = bm.prompts(cfg["vocab"], [5, 21, 1, 34, 12], seed=18)
    outs = engine.generate(prompts, SamplingParams.greedy(7))
    margin = 1e-3 if dtype == "float32" else 0.5
    for p, o in zip(prompts, outs):
        assert o.finish_reason == "length" and len(o.token_ids) == 7
        tokens = list(p)
        for got in o.token_ids:
            last = plain.forward(stored, cfg, tokens)[-1]
            best = int(torch.argmax(last))
            if got != best:
                assert float(last[best] - last[got]) < margin
            tokens.append(got)
    engine.runner.cache.check_invariants()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
def test_the_replay_program_runs_the_model(dtype_name, tmp_path_factory, tmp_path):
    folder, cfg, stored = model_case("a", dtype_name, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [40, 7, 25, 33, 18], seed=19)
    steps, peak = traces.trace_mixed(reqs, live=4, seed=3)
    out = traces.replay_program(folder, dtype_name, steps, peak, str(tmp_path / "out"),
                                cfg["vocab"])
    got = traces.collect(steps, out, cfg["vocab"])
    errors = []
    for rid, tokens in reqs.items():
        want = plain.forward(stored, cfg, tokens)
        errors += [bm.row_error(row, want[pos]) for pos, row in got[rid].items()]
    bm.judge(errors, dtype_name)


@pytest.mark.gpu
def test_the_command_line_generates_and_scores(tmp_path_factory, tmp_path, capsys):
    """``rlis generate`` picks the design by config.json and prints the plain implementation's
    greedy tokens; ``rlis perplexity`` scores a token file through the same step function."""
    from rust_llm_inference_server_amd import cli
    folder, cfg, stored = model_case("b", "float32", tmp_path_factory)
    prompt = bm.prompts(cfg["vocab"], [11], seed=20)[0]
    rc = cli.main(["generate", "--model", folder, "--dtype", "f32", "--max-seq-len", "128",
                   "--num-pages", "32", "--block-size", "8", "--max-num-seqs", "2",
                   "--max-tokens", "5", "--prompt-ids", ",".join(map(str, prompt))])
    out = capsys.readouterr()
    assert rc == 0
    got = [int(t) for t in out.out.split()]
    tokens = list(prompt)
    for g in got:
        last = plain.forward(stored, cfg, tokens)[-1]
        best = int(torch.argmax(last))
        assert g == best or float(last[best] - last[g]) < 1e-3
        tokens.append(g)
    assert len(got) == 5 and "output 5 tok (length)" in out.err
    ids = tmp_path / "ids.txt"
    ids.write_text(" ".join(map(str, bm.prompts(cfg["vocab"], [96], seed=21)[0])))
    rc = cli.main(["perplexity", "--model", folder, "--dtype", "f32", "--max-seq-len", "128",
                   "--ids-file", str(ids), "--ctx", "32"])
    out = capsys.readouterr()
    assert rc == 0 and json.loads(out.out.strip().splitlines()[-1])["ppl"] > 1.0
