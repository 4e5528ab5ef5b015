"""The Lagedra decoder in the engine against the plain implementation (``plain_lagedra.py``):
whole prompts, token-by-token decoding, portions down to two tokens, batches of unequal
requests with pages and state slots used again, long decoding, keys made to stand out far
away, at page borders and just inside and just outside every window, a far token in the
linear attention's state at the borders of its chunks, the first tokens of a sequence, and
greedy generation through the engine's scheduler.  Every case runs on the GPU (``-m gpu``,
float32 and bfloat16) and, with the kernels replaced by the slow torch double, on the CPU,
where it tests the host logic: the run order, the depth mix's slots, windows, state slots, the
convolutions' tails, the shared first values, the step layout."""
import copy
import json

import pytest
import torch

import lagedra_models as lm
import plain_lagedra as plain
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
        cfg = config if config is not None else lm.CONFIGS[name]
        w = weights if weights is not None else lm.make_weights(cfg, seed=len(name) + 7)
        store = torch.float32 if dtype == "float32" else torch.bfloat16
        folder = lm.write_folder(tmp_path_factory.mktemp(f"lagedra_{name}_{dtype}{tag}"), cfg, w,
                                 store)
        _CACHE[key] = (folder, cfg, lm.as_stored(w, store))
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
        want = lm.plain_logits(plain, cfg, stored, tokens)
        assert sorted(got[rid]) == list(range(len(tokens)))
        errors += [lm.row_error(row, want[pos]) for pos, row in got[rid].items()]
    lm.judge(errors, dtype)


# ----------------------------------------------------------------------- configuration
def test_config_round_trip_and_the_specification():
    from rust_llm_inference_server_amd.registry import architecture_of
    for cfg in lm.CONFIGS.values():
        arch = architecture_of(cfg)
        assert arch.name == "Lagedra"
        assert arch.config_to_dict(arch.parse_config(cfg)) == cfg
    spec = lm.spec_of(lm.CONFIG_A)
    names = {t.name: tuple(t.shape) for t in spec.tensor_specs()}
    # a scalar norm each in front of mixer and feed-forward; none for a layer without the latter
    assert names["l0.norm1"] == () and names["l0.norm2"] == () and "l2.norm2" not in names
    # the depth mix of layer i weighs i + 2 streams
    assert [names[f"l{i}.dwa"] for i in range(6)] == [(i + 2,) for i in range(6)]
    # sizes per layer: grouped heads, value sizes of their own, taps
    assert names["l0.mix.q"] == (64, 48) and names["l0.mix.k"] == (32, 48)
    assert names["l0.mix.v"] == (48, 48) and names["l0.mix.v.conv"] == (48, 3)
    assert names["l4.mix.q.conv"] == (48, 4) and names["l0.mix.temp"] == (4,)
    assert names["l1.mix.q"] == (72, 48) and names["l1.mix.v"] == (120, 48)
    assert names["l1.mix.norm"] == (120,) and names["l1.mlp.e5.down"] == (48, 24)
    assert names["pos"] == (512, 48) and names["head"] == (97, 48)
    # the first layer that mixes values is the others' source; a layer that mixes nothing has
    # no such tensor
    mixers = [layer.block.params["mixer"].params for layer in spec.layers]
    assert "value_mix" not in mixers[0] and "l0.mix.vmix" not in names
    assert mixers[2]["value_mix"]["source"] and not mixers[4]["value_mix"]["source"]
    assert mixers[4]["value_mix"]["key"] == mixers[5]["value_mix"]["key"]


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
    (_edit(("layers", 0, "type"), "lightning2"), "type 'lightning2'"),
    (_edit(("layers", 1, "mixer", "decay"), [0.5, 0.9]), "'decay' has 2 entries"),
    (_edit(("layers", 1, "mixer", "decay"), [0.5, 0.9, 1.5]), "'decay'"),
    (_edit(("layers", 0, "mixer", "kv_heads"), 3), "'kv_heads'"),
    (_edit(("layers", 0, "mixer", "rot", "dims"), 7), "'dims' 7"),
    (_edit(("layers", 0, "mixer", "rot", "dims"), 18), "'dims' 18"),
    (_edit(("layers", 0, "mixer", "scale"), _DROP), "'scale'"),
    (_edit(("layers", 0, "mlp", "kind"), "glu"), "kind 'glu'"),
    (_edit(("layers", 1, "mlp", "router", "groups", "count"), 4), "4 groups"),
    (_edit(("layers", 1, "mlp", "router", "top"), 5), "5 chosen"),
    (_edit(("layers", 1, "mlp", "expert", "limit"), 0.0), "'limit'"),
    (_edit(("layers", 4, "mixer", "vdim"), 16), "'v_mix'"),
    (_edit(("norm", "eps"), 0.0), "'eps'"),
    (_edit(("max_positions",), _DROP), "'max_positions'"),
])
def test_config_errors_name_the_key(edit, message):
    from rust_llm_inference_server_amd.registry import architecture_of
    cfg = copy.deepcopy(lm.CONFIG_A)
    edit(cfg)
    with pytest.raises(ConfigError) as e:
        architecture_of(cfg).parse_config(cfg)
    assert message in str(e.value)


def test_the_plain_implementation_does_not_look_ahead():
    """A position's plain logits depend on the tokens up to it and on nothing behind it; and
    they do depend on a token that has left every window (through the linear attention's
    state)."""
    cfg = lm.CONFIG_A
    stored = lm.as_stored(lm.make_weights(cfg, 5), torch.float32)
    tokens = lm.prompts(cfg["vocab"], [60], seed=1)[0]
    whole = lm.plain_logits(plain, cfg, stored, tokens)
    part = lm.plain_logits(plain, cfg, stored, tokens[:41])
    assert float((whole[:41] - part).abs().max()) < 1e-9
    other = list(tokens)
    other[3] = (other[3] + 1) % cfg["vocab"]
    assert float((lm.plain_logits(plain, cfg, stored, other)[-1] - whole[-1]).abs().max()) > 1e-6


# --------------------------------------------------------------------- the step function
@pytest.mark.parametrize("name", ["a", "b", "c", "e"])
def test_whole_prompts_and_first_tokens(backend, dtype, name, tmp_path_factory):
    folder, cfg, stored = model_case(name, dtype, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [1, 2, 3, 19, 70], seed=11)
    steps, _ = traces.trace_whole(reqs)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_decoding_token_by_token_equals_the_prompt_pass(backend, dtype, name, tmp_path_factory):
    """One request decoded from its first token on (the convolutions' zeros in front of the
    sequence, then their tails), one after a prompt, so that every window passes over decoded
    tokens; single tokens go through captured steps on the GPU."""
    folder, cfg, stored = model_case(name, dtype, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [45, 80], seed=12)
    ids = list(reqs)
    steps, _ = traces.trace_tail({ids[0]: reqs[ids[0]]}, tail=44)
    more, _ = traces.trace_tail({ids[1]: reqs[ids[1]]}, tail=45)
    for s in more:
        s["step"] += len(steps)
    check_trace(runner_for(folder, backend, dtype), steps + more, reqs, cfg, stored, dtype)


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_portions_of_any_size(backend, dtype, name, tmp_path_factory):
    """Portions of 7, 2, 16, 3, 24, 2, 33, ... tokens: tails shorter than the taps, portions
    that end inside a page and inside a window."""
    folder, cfg, stored = model_case(name, dtype, tmp_path_factory)
    reqs = traces.random_requests(cfg["vocab"], [90, 37], seed=13)
    steps, _ = traces.trace_portions(reqs)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


@pytest.mark.parametrize("name", ["a", "b", "c", "e"])
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
    lm.judge([lm.row_error(row, alone[rid][pos]) for rid in reqs
              for pos, row in together[rid].items()], dtype)


@pytest.mark.parametrize("name", ["a", "b"])
def test_long_prompts_and_long_decoding(backend, dtype, name, tmp_path_factory):
    """A prompt of hundreds of tokens in one step (the linear attention's chunked form where
    the engine has one), then hundreds of single-token steps: the states are carried, never
    rebuilt, windows move over many pages (which are given back), and what the first tokens
    wrote still counts at the end (decays of 0.999 and of 1)."""
    folder, cfg, stored = model_case(name, dtype, tmp_path_factory)
    n, tail = (150, 60) if backend.type == "cpu" else (390, 150)
    reqs = traces.random_requests(cfg["vocab"], [n], seed=16)
    steps, _ = traces.trace_tail(reqs, tail=tail)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


def test_prompts_of_hundreds_of_tokens_at_head_sizes_of_real_models(backend, dtype,
                                                                    tmp_path_factory):
    """Heads of 64 and 128: whole prompts of up to 700 tokens in one step (the linear
    attention's chunks, the attention kernels' tiles of 64 and 128 queries, the rotation inside
    the attention kernel where the whole head of 64 turns), the same prompts with their ends
    decoded, and in portions beside each other."""
    folder, cfg, stored = model_case("d", dtype, tmp_path_factory)
    lengths = [300, 130] if backend.type == "cpu" else [700, 300, 130, 257]
    reqs = traces.random_requests(cfg["vocab"], lengths, seed=71)
    make = lambda: runner_for(folder, backend, dtype, num_pages=130, max_positions=1024)
    steps, _ = traces.trace_whole(reqs)
    check_trace(make(), steps, reqs, cfg, stored, dtype)
    steps, _ = traces.trace_tail(reqs, tail=20)
    check_trace(make(), steps, reqs, cfg, stored, dtype)
    steps, peak = traces.trace_mixed(reqs, live=3, seed=6)
    check_trace(runner_for(folder, backend, dtype, num_pages=-(-peak // 16), max_num_seqs=3,
                           max_positions=1024), steps, reqs, cfg, stored, dtype)
    # a long portion beside single decoded tokens of two other requests, in one step
    reqs = traces.random_requests(cfg["vocab"], [60, 70, 330], seed=72)
    cuts = [{"r0": (0, 40), "r1": (0, 50)}, {"r0": (40, 41), "r1": (50, 51), "r2": (0, 300)},
            {"r0": (41, 60), "r1": (51, 70), "r2": (300, 330)}]
    steps = [{"step": i, "end": [], "entries": [
        {"id": rid, "tokens": reqs[rid][lo:hi], "want": list(range(hi - lo))}
        for rid, (lo, hi) in cut.items()]} for i, cut in enumerate(cuts)]
    steps[-1]["end"] = ["r0", "r1", "r2"]
    check_trace(make(), steps, reqs, cfg, stored, dtype)


# ------------------------------------------------------------- keys made to stand out
KEY_TOKEN, QUERY_TOKEN, FILL_TOKEN = 5, 9, 1


def _marked(cfg, seed):
    """Weights in which coordinate 0 of the stream is nonzero at ``KEY_TOKEN`` only and
    coordinate 1 at ``QUERY_TOKEN`` only, in every layer: the embedding sets them, no position
    vector and no layer's output touches them, and the depth mixes weigh them positively."""
    w = lm.make_weights(cfg, seed=seed)
    w["embed"][:, :2] = 0.0
    w["embed"][KEY_TOKEN, 0] = 3.0
    w["embed"][QUERY_TOKEN, 1] = 3.0
    w["pos"][:, :2] = 0.0
    for name, t in w.items():
        last = name.split(".")[-1]
        if last in ("o", "down"):
            t[:2] = 0.0
        elif last == "dwa":
            t.abs_().clamp_(min=0.2)
        elif last in ("norm1", "norm2"):
            t.abs_().clamp_(min=0.5)
    return w


def _attention_stands_out(cfg, w, layer, boost=8.0):
    """In every head of ``layer``'s attention the key of ``KEY_TOKEN`` gets the cap's score from
    a query of ``QUERY_TOKEN``: one channel of every key head reads stream coordinate 0, the
    same channel of every query head coordinate 1, through taps that pass the current token
    alone.  The channel is one that is not rotated, or else the slowest rotated pair's first
    half (whose partner is emptied, so that the product falls only by the cosine of a small
    angle)."""
    m = cfg["layers"][layer]["mixer"]
    p = f"l{layer}.mix"
    d, dims = m["dim"], m["rot"]["dims"]
    chans = [dims] if dims < d else [dims // 2 - 1, dims - 1]
    for name, heads in (("q", m["heads"]), ("k", m["kv_heads"])):
        for head in range(heads):
            for n, c in enumerate(chans):
                row = head * d + c
                w[f"{p}.{name}"][row] = 0.0
                if n == 0:
                    w[f"{p}.{name}"][row, 1 if name == "q" else 0] = boost
                w[f"{p}.{name}.conv"][row] = 0.0
                w[f"{p}.{name}.conv"][row, -1] = 1.0
    w[p + ".temp"].clamp_(min=1.0)
    m["softcap"] = max(m["softcap"], 12.0)       # far above what hundreds of other keys add up to
    return w


def _tokens(vocab, n, seed):
    return [t if t not in (KEY_TOKEN, QUERY_TOKEN) else FILL_TOKEN
            for t in lm.prompts(vocab, [n], seed=seed)[0]]


@pytest.mark.parametrize("layer, back", [(0, 19), (0, 20), (2, 15), (2, 16), (4, 32), (4, 33),
                                         (5, 199), (5, 200)])
def test_keys_just_inside_and_outside_every_window(backend, dtype, layer, back,
                                                   tmp_path_factory):
    """Windows of 20, 16 (a page), 33 and 200 positions.  A key that stands out lies ``back``
    positions behind the query: the last one inside or the first one outside.  A window that is
    one token off, in a prompt's portion or decoded alone, moves the row far."""
    cfg = copy.deepcopy(lm.CONFIG_A)
    size = cfg["layers"][layer]["mixer"]["mask"]["size"]
    w = _attention_stands_out(cfg, _marked(cfg, seed=31 + layer), layer)
    folder, _, stored = model_case("a", dtype, tmp_path_factory, weights=w,
                                   tag=f"edge{layer}", config=cfg)
    n = back + 70
    tokens = _tokens(cfg["vocab"], n, seed=32)
    queries = (back + 25, n - 4)                 # one in the prompt's part, one decoded
    for query in queries:
        tokens[query] = QUERY_TOKEN
        tokens[query - back] = KEY_TOKEN
    # the construction works: with the window one position off (shorter when the key is the
    # last one inside, longer when it is the first one outside) the plain logits move far
    other = copy.deepcopy(cfg)
    other["layers"][layer]["mixer"]["mask"]["size"] += -1 if back == size - 1 else 1
    a, b = lm.plain_logits(plain, cfg, stored, tokens), lm.plain_logits(plain, other, stored, tokens)
    for query in queries:
        assert lm.row_error(a[query], b[query]) > 0.03
    reqs = {"r": tokens}
    steps, _ = traces.trace_tail(reqs, tail=12)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)
    steps, _ = traces.trace_portions(reqs)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


@pytest.mark.parametrize("far", [0, 15, 16, 17, 48])
def test_a_far_key_that_stands_out(backend, dtype, far, tmp_path_factory):
    """A window of 200 over pages of 16: the token at ``far`` (a page's first or last position
    among them) takes most of the weight of queries 150 and more positions on, in a prompt's
    portion and decoded alone.  Were its row lost or read from a wrong page, the layer would
    return another token's value."""
    cfg = copy.deepcopy(lm.CONFIG_A)
    w = _attention_stands_out(cfg, _marked(cfg, seed=41), 5)
    folder, _, stored = model_case("a", dtype, tmp_path_factory, weights=w, tag="far", config=cfg)
    tokens = _tokens(cfg["vocab"], 200, seed=42)
    tokens[far] = KEY_TOKEN
    tokens[far + 140] = tokens[197] = QUERY_TOKEN
    moved = list(tokens)
    moved[far] = FILL_TOKEN
    a, b = lm.plain_logits(plain, cfg, stored, tokens), lm.plain_logits(plain, cfg, stored, moved)
    assert lm.row_error(a[far + 140], b[far + 140]) > 0.03 and lm.row_error(a[197], b[197]) > 0.03
    reqs = {"r": tokens}
    steps, _ = traces.trace_tail(reqs, tail=6)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


@pytest.mark.parametrize("far", [0, 63, 64, 65, 127, 128])
def test_a_far_token_in_the_linear_attention_state(backend, dtype, far, tmp_path_factory):
    """A head that forgets nothing (decay 1): one key channel is filled by ``KEY_TOKEN`` alone
    and asked for by ``QUERY_TOKEN`` alone, hundreds of positions later, so that the read-out
    is that token's value or nearly nothing.  ``far`` is the first or last token of a chunk of
    64 among them; the queries lie in a prompt's portion and among decoded tokens."""
    cfg = copy.deepcopy(lm.CONFIG_A)
    w = _marked(cfg, seed=51)
    m = cfg["layers"][3]["mixer"]
    assert m["decay"][0] == 1.0
    for name, col in (("q", 1), ("k", 0)):
        w[f"l3.mix.{name}"][0] = 0.0
        w[f"l3.mix.{name}"][0, col] = 6.0
    folder, _, stored = model_case("a", dtype, tmp_path_factory, weights=w, tag="state", config=cfg)
    n = 330
    tokens = _tokens(cfg["vocab"], n, seed=52)
    tokens[far] = KEY_TOKEN
    tokens[290] = tokens[n - 3] = QUERY_TOKEN
    moved = list(tokens)
    moved[far] = FILL_TOKEN
    a, b = lm.plain_logits(plain, cfg, stored, tokens), lm.plain_logits(plain, cfg, stored, moved)
    assert lm.row_error(a[290], b[290]) > 0.03 and lm.row_error(a[n - 3], b[n - 3]) > 0.03
    reqs = {"r": tokens}
    steps, _ = traces.trace_tail(reqs, tail=8)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)
    # the same prompt cut at a chunk's border and one token to either side of it
    steps = [{"step": i, "entries": [{"id": "r", "tokens": tokens[lo:hi],
                                      "want": list(range(hi - lo))}], "end": []}
             for i, (lo, hi) in enumerate([(0, 63), (63, 65), (65, 193), (193, n)])]
    steps[-1]["end"] = ["r"]
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


def test_scores_reach_the_cap(backend, dtype, tmp_path_factory):
    """Queries and keys ten times as large: most scores lie on the flat part of the cap, where
    an engine without it (or with the cap in front of the head's number) is far off."""
    cfg = lm.CONFIG_C
    w = lm.make_weights(cfg, seed=61)
    for i in range(3):
        w[f"l{i}.mix.q"] *= 10.0
    folder, _, stored = model_case("c", dtype, tmp_path_factory, weights=w, tag="cap")
    reqs = traces.random_requests(cfg["vocab"], [40], seed=62)
    loose = copy.deepcopy(cfg)
    for layer in loose["layers"]:
        layer["mixer"]["softcap"] *= 3.0
    tokens = reqs["r0"]
    assert lm.row_error(lm.plain_logits(plain, cfg, stored, tokens)[-1],
                        lm.plain_logits(plain, loose, stored, tokens)[-1]) > 0.05
    steps, _ = traces.trace_tail(reqs, tail=5)
    check_trace(runner_for(folder, backend, dtype), steps, reqs, cfg, stored, dtype)


def test_a_state_slot_is_cleared_for_its_next_request(backend, dtype, tmp_path_factory):
    """One slot, requests one after the other: each starts from a zero state and from zeros in
    front of its convolutions, not from what the one before left."""
    for name in ("a", "b"):
        folder, cfg, stored = model_case(name, dtype, tmp_path_factory)
        reqs = traces.random_requests(cfg["vocab"], [30, 12, 3], seed=17)
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
    prompts = lm.prompts(cfg["vocab"], [5, 21, 1, 34, 12], seed=18)
    outs = engine.generate(prompts, SamplingParams.greedy(7))
    margin = 1e-3 if dtype == "float32" else 0.5
    for p, o in zip(prompts, outs):
        assert o.finish_reason == "length" and len(o.token_ids) == 7
        tokens = list(p)
        for got in o.token_ids:
            last = lm.plain_logits(plain, cfg, stored, tokens)[-1]
            best = int(torch.argmax(last))
            if got != best:
                assert float(last[best] - last[got]) < margin
            tokens.append(got)
    engine.runner.cache.check_invariants()


def test_positions_beyond_the_table_are_refused(backend, tmp_path_factory):
    """The design has a vector per position up to ``max_positions``: the loaded model's longest
    sequence is that many, and a longer one is an error, not a read past the table."""
    from rust_llm_inference_server_amd.engine import ModelRunner, StepEntry, load_model
    folder, cfg, _ = model_case("c", "float32", tmp_path_factory)
    rows = cfg["max_positions"]
    model = load_model(folder, "float32", rows + 100, backend)
    assert model.max_positions == rows
    runner = ModelRunner(model, num_pages=-(-rows // 16) + 2, page_size=16, max_num_seqs=1)
    with pytest.raises(ValueError):
        runner.reserve(0, rows + 1)
    runner.reserve(0, rows)
    out = runner.step([StepEntry(0, lm.prompts(cfg["vocab"], [rows], seed=3)[0], [rows - 1])])
    assert out.shape == (1, cfg["vocab"]) and bool(torch.isfinite(out).all())


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
        want = lm.plain_logits(plain, cfg, stored, tokens)
        errors += [lm.row_error(row, want[pos]) for pos, row in got[rid].items()]
    lm.judge(errors, dtype_name)


@pytest.mark.gpu
def test_the_command_line_generates_and_scores(tmp_path_factory, tmp_path, capsys):
    """``rlis generate`` picks the design by config.json and prints the plain implementation's
    greedy tokens; ``rlis perplexity`` scores a token file through the same step function."""
    from rust_llm_inference_server_amd import cli
    folder, cfg, stored = model_case("b", "float32", tmp_path_factory)
    prompt = lm.prompts(cfg["vocab"], [11], seed=20)[0]
    rc = cli.main(["generate", "--model", folder, "--dtype", "f32", "--max-seq-len", "128",
                   "--num-pages", "32", "--block-size", "8", "--max-num-seqs", "2",
                   "--max-tokens", "5", "--prompt-ids", ",".join(map(str, prompt))])
    out = capsys.readouterr()
    assert rc == 0
    got = [int(t) for t in out.out.split()]
    tokens = list(prompt)
    for g in got:
        last = lm.plain_logits(plain, cfg, stored, tokens)[-1]
        best = int(torch.argmax(last))
        assert g == best or float(last[best] - last[g]) < 1e-3
        tokens.append(g)
    assert len(got) == 5 and "output 5 tok (length)" in out.err
    ids = tmp_path / "ids.txt"
    ids.write_text(" ".join(map(str, lm.prompts(cfg["vocab"], [96], seed=21)[0])))
    rc = cli.main(["perplexity", "--model", folder, "--dtype", "f32", "--max-seq-len", "128",
                   "--ids-file", str(ids), "--ctx", "32"])
    out = capsys.readouterr()
    assert rc == 0 and json.loads(out.out.strip().splitlines()[-1])["ppl"] > 1.0
