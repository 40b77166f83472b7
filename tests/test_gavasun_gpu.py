"""Gavasun through the engine against the plain implementation: every mechanism alone, and every
way of cutting, batching and reusing that must not change the logits."""

import pytest
import torch

pytestmark = pytest.mark.gpu

import burn_transformers_amd as bt  # noqa: E402
import plain_gavasun as plain  # noqa: E402
from burn_transformers_amd.cache.ledger import RELEASED  # noqa: E402
from gavasun_helpers import (CONFIGS, attention, config_for, engine_for, latent, layer, model_config, model_for, plain_logits,  # noqa: E402
                             prompts_for, random_config, rotation, tolerance, weights_for)

DTYPES = ["float32", "bfloat16"]
SHARPEN = 4.0        # factor on the scales of the queries' norms where attention is to put its weight on few keys


def check(got, want, dtype, what):
    """float32: every row within the bound.  bfloat16 (whose runs make no choice of experts that could hang on a
    close call, see ``gavasun_helpers.config_for``): a row in forty (at least two) may pass the bound: the norm of a
    head's read-out divides by the read-out's own size, so where a read-out is nearly zero, rounding to 8 bits
    decides its direction."""
    got = got.detach().cpu().double()
    assert torch.isfinite(got).all(), what
    rows = (got - want).abs().max(dim=1).values
    bound = tolerance(dtype, want)
    over = int((rows > bound).sum())
    allowed = 0 if dtype == "float32" else max(2, rows.numel() // 40)
    assert over <= allowed, f"{what}: {over} rows over {bound}, max abs error {float(rows.max())}"


def whole(engine, ids):
    slot = engine.open()
    logits = engine.step([(slot, ids)], want=[list(range(len(ids)))]).clone()
    engine.close(slot)
    return logits


def decoded(engine, ids, head):
    """The first ``head`` tokens in one step, the others one by one."""
    slot = engine.open()
    rows = [engine.step([(slot, ids[:head])], want=[list(range(head))]).clone()]
    rows += [engine.step([(slot, [token])]).clone() for token in ids[head:]]
    engine.close(slot)
    return torch.cat(rows)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,lengths", [("attention", [1, 2, 39, 40, 41, 64, 65, 130]), ("latent", [1, 2, 32, 33, 34, 64, 65, 130]),
                                          ("delta", [1, 2, 3, 4, 5, 70, 200]), ("dense", [1, 17, 80]),
                                          ("experts", [1, 2, 33, 90]), ("basic", [1, 2, 23, 24, 25, 49, 130]),
                                          ("odd", [1, 6, 7, 8, 99, 101, 210]), ("narrow_latent", [1, 50, 100]),
                                          ("wide_heads", [1, 31, 90]), ("unaligned", [1, 2, 10, 70])])
def test_each_mechanism_and_each_request_whole(name, dtype, lengths):
    engine = engine_for(name, dtype)
    for ids in prompts_for(name, lengths):
        check(whole(engine, ids), plain_logits(name, ids, dtype=dtype), dtype, f"{name} whole {len(ids)}")
    engine.cache.ledger.check()


def test_residual_stream_after_every_run_of_a_layer():
    """The stream itself, run by run (the looped layers twice), in float32."""
    name = "basic"
    model = model_for(name, "float32")
    engine = bt.Engine(model, max_tokens=256, graphs=False, programs=False)
    ids = prompts_for(name, [29], seed=4)[0]
    want = []
    plain.forward(ids, weights_for(name), CONFIGS[name][0], streams=want)
    caught, restore = [], []
    for block in model.blocks:
        restore.append(block)

        def run(stream, step, memory, forward=block.forward):
            forward(stream, step, memory)
            stream.flush()
            caught.append(stream.x.detach().cpu().double().clone())
        block.forward = run
    try:
        slot = engine.open()
        engine.step([(slot, ids)])
        engine.close(slot)
    finally:
        for block in restore:
            del block.forward
    assert len(caught) == len(want) == 6
    for number, (got, reference) in enumerate(zip(caught, want)):
        assert float((got - reference).abs().max()) <= 2e-5 + 2e-5 * float(reference.abs().max()), f"run {number}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,length,tail", [("basic", 80, 40), ("odd", 110, 20), ("attention", 140, 90), ("latent", 140, 80),
                                              ("delta", 9, 8), ("narrow_latent", 130, 75), ("wide_heads", 100, 70), ("unaligned", 30, 20)])
def test_prompt_then_token_by_token(name, dtype, length, tail):
    """The last tokens one by one through the cache and the state give what the whole prompt gives; the tails
    let windows pass over decoded tokens and chunks begin among them."""
    engine = engine_for(name, dtype)
    ids = prompts_for(name, [length], seed=3)[0]
    check(decoded(engine, ids, length - tail), plain_logits(name, ids, dtype=dtype), dtype, f"{name} decode")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["basic", "odd"])
def test_from_the_first_token_one_by_one(name, dtype):
    """The first tokens of a sequence: the convolutions read zeros before the start, windows and chunks are not
    full, the state starts at zero."""
    engine = engine_for(name, dtype)
    ids = prompts_for(name, [60], seed=9)[0]
    check(decoded(engine, ids, 1), plain_logits(name, ids, dtype=dtype), dtype, f"{name} from the first token")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,portion", [("basic", 2), ("basic", 3), ("basic", 24), ("basic", 64), ("basic", 65),
                                          ("odd", 2), ("odd", 7), ("odd", 50), ("long", 193)])
def test_prompt_in_portions(name, dtype, portion):
    """Portions that start anywhere in a window, a chunk and a block; portions shorter than the convolutions' taps."""
    engine = engine_for(name, dtype)
    ids = prompts_for(name, [600 if name == "long" else 151], seed=5)[0]
    slot = engine.open()
    rows = []
    for at in range(0, len(ids), portion):
        part = ids[at:at + portion]
        rows.append(engine.step([(slot, part)], want=[list(range(len(part)))]).clone())
    check(torch.cat(rows), plain_logits(name, ids, dtype=dtype), dtype, f"{name} in portions of {portion}")
    engine.close(slot)
    engine.cache.ledger.check()


def batch_then_decode(engine, prompts, extra):
    """The prompts in one step, then one token of every request that still has some in each further step."""
    slots = [engine.open() for _ in prompts]
    got = [[] for _ in prompts]
    logits = engine.step(list(zip(slots, prompts)), want=[list(range(len(p))) for p in prompts])
    at = 0
    for i, p in enumerate(prompts):
        got[i].append(logits[at:at + len(p)].clone())
        at += len(p)
    for t in range(max(len(e) for e in extra)):
        live = [i for i in range(len(prompts)) if t < len(extra[i])]
        logits = engine.step([(slots[i], [extra[i][t]]) for i in live])
        for row, i in enumerate(live):
            got[i].append(logits[row:row + 1].clone())
        for i in range(len(prompts)):
            if t + 1 == len(extra[i]):
                engine.close(slots[i])
    return [torch.cat(rows) for rows in got]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["basic", "odd"])
def test_unequal_batch_decoded_together_then_slots_and_blocks_reused(name, dtype):
    """Requests of unequal length in one step, decoded together while the shorter ones end; then a
    second batch in the slots, blocks and state rows the first gave back."""
    engine = engine_for(name, dtype, max_tokens=1024)
    for number, lengths in enumerate([[1, 70, 33, 129], [64, 5, 90]]):
        prompts = prompts_for(name, lengths, seed=20 + number)
        extra = [prompts_for(name, [t], seed=30 + i)[0] for i, t in enumerate([12, 5, 9, 3][:len(prompts)])]
        for i, got in enumerate(batch_then_decode(engine, prompts, extra)):
            check(got, plain_logits(name, prompts[i] + extra[i], dtype=dtype), dtype, f"{name} batch {number} request {i}")
        engine.cache.ledger.check()
    assert not engine.cache.ledger.live_slots()


@pytest.mark.parametrize("dtype", DTYPES)
def test_chunks_and_windows_over_several_blocks_whole_and_decoded(dtype):
    """Attention sharpened so that weight lies on single keys: a chunk of 200 and a window of 150 positions span
    several blocks of the cache; whole, and decoded while the window's first key passes a block border and a chunk
    begins among the decoded tokens."""
    name = "long"
    ids = prompts_for(name, [700], seed=11)[0]
    want = plain_logits(name, ids, SHARPEN, dtype)
    engine = engine_for(name, dtype, sharpen=SHARPEN)
    check(whole(engine, ids), want, dtype, "long whole")
    slot = engine.open()
    head = 560                      # position 600 begins a chunk; the window's first key passes position 448 at token 597
    rows = [engine.step([(slot, ids[:head])], want=[list(range(head))]).clone()]
    rows += [engine.step([(slot, [token])]).clone() for token in ids[head:]]
    check(torch.cat(rows), want, dtype, "long decoded across a chunk's start and a block border")
    held = [engine.cache.blocks(slot, group) for group in range(len(engine.cache.kv_groups))]
    engine.close(slot)
    assert any(RELEASED in blocks for blocks in held)       # blocks behind the window and the chunk went back meanwhile


def test_sharpened_attention_puts_weight_near_the_edges():
    """The premise of the test above, on the plain implementation: with the sharpened queries, a window or a chunk
    that is half as long moves the last logits by several times the widest bound here."""
    name = "long"
    config = CONFIGS[name][0]
    ids = prompts_for(name, [440], seed=11)[0]
    weights = weights_for(name, SHARPEN)
    full = plain.forward(ids, weights, config)[-1]
    for index, size in ((0, 100), (1, 75)):
        layers = list(config["layers"])
        layers[index] = dict(layers[index], mixer=dict(layers[index]["mixer"], mask={"size": size}))
        moved = plain.forward(ids, weights, dict(config, layers=layers))[-1]
        assert float((full - moved).abs().max()) > 4 * tolerance("bfloat16", full)


EDGE_CHUNK = model_config([layer(attention(2, 1, 32, 32, 0.18, taps=3, rot=rotation(16, 100.0), chunk=70))], vocab=83)
EDGE_WINDOW = model_config([layer(latent(2, 32, 16, 32, 40, 48, 0.15, base=100.0, window=70))], vocab=83)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["chunk", "window"])
@pytest.mark.parametrize("how", ["whole", "decoded"])
def test_the_last_key_seen_and_the_first_not_seen(kind, dtype, how):
    """One layer, so that a token reaches a later position only as a key that position sees (scores of a size that
    spreads a query's weight over all its keys).  Changing the token just inside the edge moves the logits there;
    changing the one just outside leaves every bit as it was.  (The
    chunk attention's keys pass a convolution of three taps: a token is part of the keys of the next two positions.)
    The edges lie at positions that are no block border (a chunk begins at 140; the window of 70 begins at 131 for
    the query at 200) and at one that is (the window begins at 128 for the query at 197, 64 for 133)."""
    config = EDGE_CHUNK if kind == "chunk" else EDGE_WINDOW
    _, tensors = bt.random_tensors(config, 17)
    stored = {k: v.to(torch.bfloat16) for k, v in tensors.items()}
    engine = bt.Engine(bt.model_from_tensors(config, stored, dtype, "cuda:0"), max_tokens=1024)
    ids = torch.randint(0, config["vocab"], (210,), generator=torch.Generator().manual_seed(3)).tolist()
    run = (lambda tokens: whole(engine, tokens)) if how == "whole" else (lambda tokens: decoded(engine, tokens, 120))
    base = run(ids)
    cases = [(200, 138, 137), (141, 138, 137)] if kind == "chunk" else [(200, 131, 130), (197, 128, 127), (133, 64, 63)]
    for query, inside, outside in cases:
        for place, seen in ((inside, True), (outside, False)):
            other = list(ids)
            other[place] = (other[place] + 1) % config["vocab"]
            moved = (run(other)[query] - base[query]).abs().max().item()
            if seen:
                assert moved > 1e-4, f"{kind}: the token at {place} should reach position {query}"
            else:
                assert moved == 0.0, f"{kind}: the token at {place} must not reach position {query}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(dtype):
    name = "basic"
    engine = engine_for(name, dtype)
    ids = prompts_for(name, [330], seed=12)[0]
    check(decoded(engine, ids, 4), plain_logits(name, ids, dtype=dtype), dtype, "300 tokens one by one")


def test_a_state_row_that_is_used_again_starts_at_zero():
    """A slot that held a long sequence is given to a new one: its states and the convolutions' inputs are
    cleared, its blocks are others'."""
    name = "basic"
    engine = engine_for(name, "float32", max_tokens=512)
    first, second = prompts_for(name, [200, 30], seed=40)
    slot = engine.open()
    engine.step([(slot, first)])
    engine.close(slot)
    again = engine.open()
    assert again == slot
    got = engine.step([(again, second)], want=[list(range(len(second)))]).clone()
    engine.close(again)
    check(got, plain_logits(name, second), "float32", "a slot used again")


@pytest.mark.parametrize("seed", range(12))
def test_configurations_drawn_at_random(seed):
    """Layers, sizes, loops and constants drawn from a seed: three unequal prompts in one step, then decoded together
    while the shorter requests end; float32, and bfloat16 for every other seed (there every token uses every expert)."""
    config = random_config(seed)
    _, tensors = bt.random_tensors(config, seed)
    stored = {k: v.to(torch.bfloat16) for k, v in tensors.items()}
    weights = {k: v.float() for k, v in stored.items()}
    gen = torch.Generator().manual_seed(seed)
    prompts = [torch.randint(0, config["vocab"], (n,), generator=gen).tolist() for n in (3, 70, 200)]
    extra = [torch.randint(0, config["vocab"], (t,), generator=gen).tolist() for t in (4, 9, 6)]
    for dtype in DTYPES[:1 + seed % 2]:
        used = config
        if dtype == "bfloat16":
            used = dict(config, layers=[dict(e, mlp=dict(e["mlp"], router=dict(e["mlp"]["router"], top=e["mlp"]["router"]["experts"])))
                                        if e["mlp"] and e["mlp"]["kind"] == "moe" else e for e in config["layers"]])
        engine = bt.Engine(bt.model_from_tensors(used, stored, dtype, "cuda:0"), max_tokens=1024)
        for i, got in enumerate(batch_then_decode(engine, prompts, extra)):
            check(got, plain.forward(prompts[i] + extra[i], weights, used), dtype, f"seed {seed} request {i} {dtype}: {config}")


@pytest.mark.parametrize("graphs,programs", [(False, False), (False, True), ("always", True)])
def test_launch_lists_and_graphs_give_the_same_bits(graphs, programs):
    name = "basic"
    ids = prompts_for(name, [70], seed=13)[0]
    rows = {}
    for key, options in (("direct", dict(graphs=False, programs=False)), ("other", dict(graphs=graphs, programs=programs))):
        engine = engine_for(name, "bfloat16", **options)
        got = []
        for _ in range(3):          # a shape comes again: recorded, then replayed
            slot = engine.open()
            got.append(engine.step([(slot, ids[:50])], want=[[49]]).clone())
            got += [engine.step([(slot, [token])]).clone() for token in ids[50:]]
            engine.close(slot)
        rows[key] = torch.cat(got)
    assert torch.equal(rows["direct"], rows["other"])


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_entry_point(dtype):
    name = "basic"
    config = config_for(name, dtype)
    prompts = prompts_for(name, [5, 40, 1, 27], seed=14)
    engine = engine_for(name, dtype)
    got = bt.generate(engine, prompts, bt.GenerationConfig(max_new_tokens=10), prefill_chunk=16)
    for prompt, sequence in zip(prompts, got):
        ids = list(prompt)
        for token in sequence.token_ids:
            logits = plain.forward(ids, weights_for(name), config)[-1]
            best = int(logits.argmax())
            if dtype == "float32":
                assert token == best
            else:                    # 8-bit operands may take a token whose logit is within rounding of the best
                assert float(logits[best] - logits[token]) <= tolerance(dtype, logits)
            ids.append(token)
    assert not engine.cache.ledger.live_slots()


def test_folder_round_trip_and_replay(tmp_path):
    """A folder written with random weights, loaded by what config.json names, replayed step by step."""
    import json
    import numpy as np
    from burn_transformers_amd.engine.replay import Replay, cache_tokens
    config = CONFIGS["odd"][0]
    folder = tmp_path / "model"
    weights = bt.write_random_model(str(folder), config, seed=3)
    assert json.load(open(folder / "config.json"))["architecture"] == "Gavasun"
    model = bt.load_model(str(folder), dtype="float32")
    replay = Replay(bt.Engine(model, max_tokens=cache_tokens(300)), str(tmp_path / "out"))
    a, b = prompts_for("odd", [45, 9], seed=15)
    replay.run([json.dumps({"step": 0, "entries": [{"id": "a", "tokens": a[:40], "want": [0, 39]},
                                                   {"id": "b", "tokens": b[:6], "want": [5]}], "end": []}),
                json.dumps({"step": 1, "entries": [{"id": "a", "tokens": a[40:41], "want": [0]},
                                                   {"id": "b", "tokens": b[6:7], "want": []}], "end": ["b"]}),
                json.dumps({"step": 2, "entries": [{"id": "a", "tokens": a[41:42], "want": [0]}], "end": ["a"]})],
               out=open(tmp_path / "log", "w"))
    want_a, want_b = plain.forward(a, weights, config), plain.forward(b, weights, config)
    first = torch.from_numpy(np.fromfile(tmp_path / "out" / "0.f32", dtype="<f4").reshape(3, -1)).double()
    check(first, torch.stack([want_a[0], want_a[39], want_b[5]]), "float32", "replayed step 0")
    for step, row in ((1, 40), (2, 41)):
        got = torch.from_numpy(np.fromfile(tmp_path / "out" / f"{step}.f32", dtype="<f4").reshape(1, -1)).double()
        check(got, want_a[row:row + 1], "float32", f"replayed step {step}")


def test_command_line(capsys, tmp_path):
    """The command line takes the family by config.json: random weights written from a configuration,
    then greedy tokens for two prompts, then sampled ones with the prompts fed in portions."""
    import json
    from burn_transformers_amd.cli import main
    config, seed = CONFIGS["basic"]
    cfg_path = tmp_path / "cfg.json"
    cfg_path.write_text(json.dumps(config))
    prompts = prompts_for("basic", [6, 30], seed=60)
    text = ";".join(",".join(str(t) for t in p) for p in prompts)
    assert main([str(tmp_path / "made"), text, "5", "--dtype", "float32", "--json", "--random-weights", str(cfg_path),
                 "--weights-seed", str(seed)]) == 0
    lines = [json.loads(line) for line in capsys.readouterr().out.strip().splitlines()]
    weights = weights_for("basic")
    assert [line["token_ids"] for line in lines] == [plain.greedy(p, weights, config, 5) for p in prompts]
    assert main([str(tmp_path / "made"), text, "4", "--temperature", "0.7", "--seed", "5", "--prefill-chunk-size", "4"]) == 0


def test_trace_runner_as_a_program(tmp_path):
    """bin/trace_run in a process of its own, in both number formats: a batch of two prompts, then
    both decoded together, one of them ending first."""
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    config = config_for("odd", "bfloat16")          # (no choice of experts that hangs on a close call, for both formats)
    weights = weights_for("odd")
    os.makedirs(tmp_path / "model")
    (tmp_path / "model" / "config.json").write_text(json.dumps(config))
    bt.write_safetensors(str(tmp_path / "model" / "model.safetensors"), {k: v.to(torch.bfloat16) for k, v in weights.items()})
    a, b = prompts_for("odd", [70, 12], seed=22)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": a[:66], "want": [65]}, {"id": "y", "tokens": b[:10], "want": [0, 9]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": a[66:67], "want": [0]}, {"id": "y", "tokens": b[10:11], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": a[67:68], "want": [0]}, {"id": "y", "tokens": b[11:12], "want": [0]}], "end": ["y"]},
             {"step": 3, "entries": [{"id": "x", "tokens": a[68:69], "want": [0]}], "end": ["x"]}]
    want_a, want_b = plain.forward(a, weights, config), plain.forward(b, weights, config)
    expected = {0: [want_a[65], want_b[0], want_b[9]], 1: [want_a[66]], 2: [want_a[67], want_b[11]], 3: [want_a[68]]}
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for dtype in DTYPES:
        out = tmp_path / ("out_" + dtype)
        done = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", str(tmp_path / "model"),
                               "--dtype", dtype, "--out", str(out), "--max-tokens", "100"],
                              input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
        assert done.returncode == 0, done.stderr[-2000:]
        assert [line for line in done.stdout.splitlines() if line.startswith("done")] == [f"done {i}" for i in range(4)]
        for step, rows in expected.items():
            got = torch.from_numpy(np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(len(rows), -1)).double()
            want = torch.stack(rows)
            bound = tolerance(dtype, want_a)
            assert float((got - want).abs().max()) <= bound, (dtype, step)
