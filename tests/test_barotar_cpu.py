"""Barotar through the engine's own step function, cache manager, scheduler and entry point on the CPU (torch twins
of the kernels) against the plain implementation: configuration and weights, each mechanism, every way of cutting
and batching, pages and state slots used again, windows' edges, far keys, and greedy generation."""
import io
import json
import os
import tempfile

import numpy as np
import pytest
import torch

import plain_barotar as plain
import traces
from helpers import random_tokens
from llmserver_amd.config import ConfigError, UnsupportedModelError, config_from_dict
from llmserver_amd.engine.batch import StepEntry
from llmserver_amd.engine.replay import make_runner, replay
from llmserver_amd.parts import PagedAndStateSpec, StateSpec
from llmserver_amd.weights import WeightsError, build_model
from tiny_barotar import BA, BB, BC, CASES, model_folder, plain_logits, plain_model
from torch_ops import TorchOps


def runner_for(case, max_tokens, page=None, live=4):
    return make_runner(model_folder(case), "float32", max_tokens, page or CASES[case][2], device="cpu", ops=TorchOps(), max_live=live)


def run(case, steps, tmp_path, page=None):
    runner = runner_for(case, traces.peak_tokens(steps), page)
    replay(runner, traces.to_lines(steps).splitlines(), str(tmp_path), io.StringIO())
    runner.cache.check_invariants()
    assert not runner.cache.requests and runner.cache.state_slots_free() in (None, 4)
    assert all(free == group.pool.num_pages for free, group in zip(runner.cache.available_pages(), runner.cache.groups))
    return traces.collect(steps, str(tmp_path), CASES[case][0]["vocab"])


def check(case, results, requests, atol=1.5e-4):          # (float32 twins against float64: a few 1e-5 at most places, 8e-5 at the worst)
    for (rid, position), logits in results.items():
        expected = plain_logits(case, tuple(requests[rid]))[position].numpy()
        np.testing.assert_allclose(logits, expected, atol=atol, rtol=3e-4, err_msg=f"{case} {rid} position {position}")
    assert len(results) == sum(len(tokens) for tokens in requests.values())


def requests_of(case, lengths, seed0=300):
    return {f"q{i}": random_tokens(CASES[case][0]["vocab"], n, seed0 + i) for i, n in enumerate(lengths)}


# -- configuration and weights ---------------------------------------------------------------------------------------
def test_the_configuration_reads_back_and_refuses_what_is_not_built():
    config = config_from_dict(dict(BB))
    assert config_from_dict(config.to_dict()) == config
    assert config.layers[1].mlp is None and config.layers[0].mixer.tau == 16.0 and config.layers[1].mixer.low == 1
    assert config.layers[2].mixer.left.window == 500 and config.layers[2].mlp.keep == 4 and config.norm_eps == 1e-6
    other = json.loads(json.dumps(BA))
    other["layers"][1]["type"] = "something else"
    with pytest.raises(UnsupportedModelError, match="something else"):
        config_from_dict(other)
    other = json.loads(json.dumps(BA))
    other["layers"][1]["mlp"]["kind"] = "other"
    with pytest.raises(UnsupportedModelError, match="other"):
        config_from_dict(other)
    other = json.loads(json.dumps(BA))
    del other["layers"][0]["mixer"]["left"]["softcap"]
    with pytest.raises(ConfigError, match="softcap"):
        config_from_dict(other)
    other = json.loads(json.dumps(BA))
    other["layers"][1]["mlp"]["router"]["groups"]["count"] = 4         # six experts in four groups
    with pytest.raises(ConfigError, match="groups"):
        config_from_dict(other)
    other = json.loads(json.dumps(BA))
    other["layers"][0]["mixer"]["left"]["rot"]["dims"] = 5
    with pytest.raises(ConfigError, match="even"):
        config_from_dict(other)


def test_the_model_declares_the_checkpoints_tensors_and_its_caches():
    model = build_model(config_from_dict(dict(BA)))
    specs = model.param_specs()
    assert {"embed", "final.norm", "l0.norm1", "l0.norm1b", "l0.norm2", "l0.norm2b", "l0.mix.left.q", "l0.mix.left.q.norm", "l0.mix.left.sink",
            "l0.mix.right.mu.w", "l0.mix.right.w1", "l0.mix.right.w0", "l0.mix.right.u", "l0.mlp.gate", "l1.mix.a1", "l1.mix.a2.b",
            "l1.mix.norm", "l1.mlp.router", "l1.mlp.e5.down", "l2.mlp.e7.up"} <= set(specs)
    assert not {"l1.mlp.e6.gate", "l1.mix.left.q", "l0.mlp.router"} & set(specs)
    assert specs["l0.mix.left.q"].shape == (48, 48) and specs["l0.mix.left.v"].shape == (40, 48) and specs["l0.mix.left.o"].shape == (48, 80)
    assert specs["l0.mix.right.r"].shape == (30, 48) and specs["l0.mix.right.o"].shape == (48, 30) and specs["l0.mix.right.u"].shape == (3, 10)
    assert specs["l0.mix.right.w1"].shape == (5, 48) and specs["l1.mix.a2"].shape == (12, 3) and specs["l1.mix.norm"].shape == (9,)
    caches = model.cache_specs()
    assert isinstance(caches[0], PagedAndStateSpec) and caches[0].paged.head_dim == 32 and caches[0].paged.window == 7 and caches[0].paged.n_kv_heads == 2
    assert caches[0].state.shape == (3 * 10 * 10 + 48,) and caches[1] == StateSpec((2 * 6 * 9,), "float32")
    assert model.tie_head and model.head.param_specs().keys() <= model.ignored_names()


def test_the_inner_size_of_a_decay_comes_from_the_checkpoint_where_the_file_does_not_say(tmp_path):
    """A folder whose config.json names no inner size loads with whatever size its tensors have; a mismatch of the two
    matrices of one decay is refused."""
    from safetensors.torch import save_file
    raw, tensors = plain_model("BA")
    stripped = json.loads(json.dumps(raw))
    del stripped["layers"][0]["mixer"]["right"]["low"], stripped["layers"][1]["mixer"]["low"]
    with open(tmp_path / "config.json", "w") as handle:
        json.dump(stripped, handle)
    save_file({name: tensor.to(torch.bfloat16).contiguous() for name, tensor in tensors.items()}, str(tmp_path / "model.safetensors"))
    tokens = random_tokens(97, 30, 4)
    runner = make_runner(str(tmp_path), "float32", 64, 16, device="cpu", ops=TorchOps())
    runner.cache.open("r")
    got = runner.step([StepEntry("r", tokens, list(range(30)))]).numpy()
    np.testing.assert_allclose(got, plain_logits("BA", tuple(tokens)).numpy(), atol=5e-5, rtol=3e-4)
    assert runner.model.blocks[0].mixer.right.low == 5 and runner.model.blocks[1].mixer.low == 3
    broken = {name: tensor.to(torch.bfloat16).contiguous() for name, tensor in tensors.items()}
    broken["l1.mix.a2"] = torch.zeros(12, 4, dtype=torch.bfloat16)
    save_file(broken, str(tmp_path / "model.safetensors"))
    with pytest.raises((WeightsError, ValueError), match="inner size|wrong shapes"):
        make_runner(str(tmp_path), "float32", 64, 16, device="cpu", ops=TorchOps())


# -- schedules ---------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("case", sorted(CASES))
@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
def test_every_schedule_matches_the_plain_implementation(case, schedule, tmp_path):
    lengths = (5, 17, 33, 70, 41, 1, 64, 90, 20, 2) if schedule == "mixed" else (70, 33, 1, 2)
    requests = requests_of(case, lengths)
    if schedule == "whole":
        steps = traces.whole(requests)
    elif schedule == "tail":
        steps = traces.tail_decoded(requests, 32)
    elif schedule == "portions":
        steps = traces.changing_portions(requests, sizes=(2, 7, 1, 3, 33, 2, 2, 16, 5))
    else:
        steps = traces.mixed(requests, seed=11, budget_tokens=256)
        assert max(len(s["entries"]) for s in steps) >= 3 and sum(lengths) > traces.peak_tokens(steps)
    check(case, run(case, steps, tmp_path), requests)


def test_prefill_equals_token_by_token_decoding_from_the_first_token(tmp_path):
    """Every token alone, from position 0: states, the row before the first token, cache rows and sinks start from nothing."""
    for case in ("BA", "BB"):
        requests = requests_of(case, (40,))
        check(case, run(case, traces.tail_decoded(requests, 64), tmp_path / case), requests)


@pytest.mark.parametrize("page", [4, 8, 64])
def test_page_sizes_and_page_borders(page, tmp_path):
    requests = requests_of("BA", (2 * page + 1, page, page - 1, page + 1))
    steps = traces.changing_portions(requests, sizes=(page - 1, 2, page, 1, page + 1))
    check("BA", run("BA", steps, tmp_path, page=page), requests)


def test_state_slots_and_pages_are_used_again_in_any_order():
    """Eight requests through four slots: a slot's next holder must start from zeros, not from its predecessor's state,
    and windows give pages back while the requests still run."""
    runner = runner_for("BA", 4 * 64, live=4)
    tokens = {i: random_tokens(97, 30 + 5 * i, 900 + i) for i in range(8)}
    got = {}
    for first in (0, 4):
        live = list(range(first, first + 4))
        for rid in live:
            runner.cache.open(rid)
        assert sorted(runner.cache.record(rid).state_slot for rid in live) == [0, 1, 2, 3]
        done = {rid: 0 for rid in live}
        turn = 0
        while any(done[rid] < len(tokens[rid]) for rid in live):
            entries = []
            for rid in live[::-1] if turn % 2 else live:
                size = (1, 3, 2, 7)[(rid + turn) % 4]
                if done[rid] < len(tokens[rid]):
                    piece = tokens[rid][done[rid]:done[rid] + size]
                    entries.append(StepEntry(rid, piece, list(range(len(piece)))))
            logits = runner.step(entries)
            row = 0
            for entry in entries:
                for _ in entry.tokens:
                    got[(entry.request_id, done[entry.request_id])] = logits[row].numpy()
                    done[entry.request_id] += 1
                    row += 1
            turn += 1
        group = runner.cache.groups[0]          # the layer with a window of 7 keys: at most two pages of 16 are held
        assert all(sum(page >= 0 for page in runner.cache.record(rid).tables[group.index]) <= 2 for rid in live) and group.spec.window == 7
        for rid in live[::-1]:
            runner.cache.close(rid)
    for (rid, position), logits in got.items():
        expected = plain_logits("BA", tuple(tokens[rid]))[position].numpy()
        np.testing.assert_allclose(logits, expected, atol=5e-5, rtol=3e-4, err_msg=f"{rid} {position}")


# -- mechanisms that random weights could hide ---------------------------------------------------------------------
def sharpened(case, change):
    """The case's tensors with ``change(tensors)`` applied, written to a folder of its own; (folder, config, tensors)."""
    from safetensors.torch import save_file
    raw, tensors = plain_model(case)
    tensors = {name: tensor.clone() for name, tensor in tensors.items()}
    change(tensors)
    folder = tempfile.mkdtemp(prefix="llmserver_amd_test_sharp_")
    save_file({name: tensor.to(torch.bfloat16).contiguous() for name, tensor in tensors.items()}, os.path.join(folder, "model.safetensors"))
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    return (folder, *plain.read_folder(folder))


def logits_of(folder, tokens, cuts, page=8):
    runner = make_runner(folder, "float32", 64 * (-(-len(tokens) // 64)), page, device="cpu", ops=TorchOps())
    runner.cache.open("r")
    rows, start = [], 0
    for size in cuts:
        piece = tokens[start:start + size]
        if not piece:
            break
        rows.append(runner.step([StepEntry("r", piece, list(range(len(piece))))]).clone())
        start += len(piece)
    assert start == len(tokens)
    return torch.cat(rows).numpy()


def test_a_token_hundreds_back_decides_through_the_recurrent_state():
    """Decays pushed to one keep everything for ever: what a recurrent layer read hundreds of tokens ago decides the
    logits, in a prompt and for decoded tokens; a state that is lost, or cut off where a portion starts, shows."""
    def change(tensors):
        tensors["l0.mix.a2.b"][:] = 14.0                   # sigmoid(14)^(1/16): the state loses a millionth a token
        tensors["l1.mix.a2.b"][:] = 14.0
        tensors["l0.mix.k"] *= 3.0
    folder, raw, tensors = sharpened("BB", change)
    tokens = random_tokens(130, 300, 5)
    expected = plain.forward(raw, tensors, tokens).numpy()
    # the first tokens matter to the last logits: another start changes them
    other = plain.forward(raw, tensors, random_tokens(130, 20, 6) + tokens[20:]).numpy()
    assert np.abs(other[-1] - expected[-1]).max() > 1e-2
    for cuts in ([300], [280] + [1] * 20, [3, 150, 2, 100, 45]):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=2e-4, rtol=5e-4, err_msg=str(cuts))


def test_keys_just_inside_and_just_outside_the_window_in_prompts_and_decoding():
    """Attention made sharp and the recurrent side switched off: a layer with a window of 7 keys sees exactly the last
    seven; the oracle with a window one longer or one shorter gives other logits, so an edge that is one off shows."""
    def change(tensors):
        tensors["l0.mix.left.q"] *= 4.0
        tensors["l0.mix.left.k"] *= 4.0
        tensors["l0.mix.left.sink"][:] = -30.0
    folder, raw, tensors = sharpened("BA", change)
    raw = json.loads(json.dumps(raw))
    raw["layers"][0]["mixer"]["left"]["softcap"] = 200.0
    with open(os.path.join(folder, "config.json"), "w") as handle:
        json.dump(raw, handle)
    tokens = random_tokens(97, 90, 7)
    expected = plain.forward(raw, tensors, tokens).numpy()
    for off in (6, 8):
        wrong = json.loads(json.dumps(raw))
        wrong["layers"][0]["mixer"]["left"]["mask"]["size"] = off
        assert np.abs(plain.forward(wrong, tensors, tokens).numpy()[10:] - expected[10:]).max() > 1e-2
    for cuts in ([90], [60] + [1] * 30, [5, 2, 7, 1, 6, 8, 9, 2, 50], [7, 83], [6, 84], [8, 82]):
        for page in (4, 16):
            np.testing.assert_allclose(logits_of(folder, tokens, cuts, page), expected, atol=1e-4, rtol=5e-4, err_msg=f"{cuts} {page}")


def test_the_sink_takes_its_share_once_and_the_cap_bounds_the_scores():
    results = []
    for value in (12.0, -40.0):
        def change(tensors, value=value):
            for index in (0, 2):
                tensors[f"l{index}.mix.left.sink"][:] = value
                tensors[f"l{index}.mix.left.sink"][0] = 0.5
            tensors["l2.mix.left.q"] *= 5.0                   # scores far beyond the cap of 2: the cap decides the weights
        folder, raw, tensors = sharpened("BA", change)
        tokens = random_tokens(97, 120, 6)
        expected = plain.forward(raw, tensors, tokens).numpy()
        for cuts in ([120], [100] + [1] * 20, [2, 70, 3, 45]):
            np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=1e-4, rtol=3e-4)
        results.append(expected)
        uncapped = json.loads(json.dumps(raw))
        uncapped["layers"][2]["mixer"]["left"]["softcap"] = 1e6
        assert np.abs(plain.forward(uncapped, tensors, tokens).numpy() - expected).max() > 1e-2
    assert np.abs(results[0] - results[1]).max() > 0.05


def test_the_row_before_reaches_across_steps_and_the_bonus_counts_the_token_itself():
    """Mixing weights far from zero and one: what a token reads of the row before it decides, whatever step that row
    came in; a bonus scaled up makes the token's own key and value decide."""
    def change(tensors):
        for name in "rkvgw":
            tensors[f"l0.mix.right.mu.{name}"] = torch.linspace(-1.5, 2.5, 48, dtype=torch.float64)
        tensors["l0.mix.right.u"] *= 6.0
    folder, raw, tensors = sharpened("BA", change)
    tokens = random_tokens(97, 60, 9)
    expected = plain.forward(raw, tensors, tokens).numpy()
    assert np.abs(expected - plain.forward(*plain_model("BA"), tokens).numpy()).max() > 0.05
    for cuts in ([60], [1] * 60, [2, 1, 3, 4, 5, 1, 1, 6, 2, 35], [4, 56], [5, 55]):
        np.testing.assert_allclose(logits_of(folder, tokens, cuts), expected, atol=1e-4, rtol=3e-4, err_msg=str(cuts))


def test_router_choices_groups_and_weights_follow_the_oracle():
    """A router scaled up spreads the sigmoid scores; every token's groups and experts are the oracle's."""
    def change(tensors):
        tensors["l1.mlp.router"] *= 5.0
        tensors["l2.mlp.router"] *= 5.0
    folder, raw, tensors = sharpened("BA", change)
    tokens = random_tokens(97, 80, 12)
    np.testing.assert_allclose(logits_of(folder, tokens, [33, 2, 45]), plain.forward(raw, tensors, tokens).numpy(), atol=1e-4, rtol=3e-4)


# -- the oracle itself -------------------------------------------------------------------------------------------------
def test_the_oracles_mechanisms_by_hand():
    f64 = lambda values: torch.tensor(values, dtype=torch.float64)
    assert torch.allclose(plain.norm(f64([[3.0, 4.0]]), f64([1.0, 2.0]), 0.0), f64([[3.0, 8.0]]) / 12.5 ** 0.5)
    assert abs(float(plain.gelu_tanh(f64(1.0))) - 0.841192) < 1e-6
    quarter = plain.rotate_pairs(f64([[[1.0, 0.0, 5.0]]]), torch.tensor([1]), 10.0, 2, torch.float64)
    assert torch.allclose(quarter, f64([[[np.cos(1.0), np.sin(1.0), 5.0]]]))
    # four experts in two groups, one kept: the group with the larger sum of its two best scores wins, not the best expert's
    sizes = {"experts": 4, "top": 2, "groups": {"count": 2, "keep": 1}}
    router = f64([[2.0, 0.0], [-3.0, 0.0], [1.5, 0.0], [1.4, 0.0]])
    chosen, weights = plain.route(f64([[1.0, 0.0]]), router, sizes)
    assert chosen.tolist() == [[2, 3]] and torch.allclose(weights, torch.sigmoid(f64([[1.5, 1.4]])), atol=1e-6)
    # one token through an expert by hand: the gate is clamped from above only, the up projection from both sides
    tensors = {"e.gate": f64([[3.0], [-3.0]]), "e.up": f64([[-5.0], [0.5]]), "e.down": f64([[1.0, 1.0]])}
    g = np.array([1.0, -3.0])
    by_hand = float((g / (1 + np.exp(-1.702 * g)) * (np.array([-1.0, 0.5]) + 1)).sum())
    assert abs(float(plain.expert(f64([[1.0]]), tensors, "e.", 1.0)) - by_hand) < 1e-12
    # the recurrence by hand, one head of one channel: logit 0 and tau 1 halve the state at every token; keys and values
    # of one; the gate's input of 1 gives silu(1); without the norm's weight the read-outs would be 1, 1.5, 1.75
    one = f64([[1.0]])
    t = {"p.q": one, "p.k": one, "p.v": one, "p.g": one, "p.o": one, "p.norm": f64([2.0]), "p.a1": one * 0, "p.a2": one * 0, "p.a2.b": f64([0.0])}
    out = plain.gated_linear_attention(torch.ones(3, 1, dtype=torch.float64), t, "p.", {"heads": 1, "dim": 1, "vdim": 1, "tau": 1.0}, 0.0)
    assert torch.allclose(out, 2.0 * float(plain.silu(f64(1.0))) * torch.ones(3, 1, dtype=torch.float64))      # (a norm over one number leaves its sign)
    t = {"p.r": one, "p.k": one, "p.v": one, "p.g": one, "p.o": one, "p.norm": f64([1.0]), "p.w1": one * 0, "p.w2": one * 0, "p.w0": f64([0.0]),
         "p.u": f64([[3.0]]), **{f"p.mu.{name}": f64([0.0]) for name in "rkvgw"}}
    # (S + u k v) r with the bonus u = 3, divided by its own size: the unit norm leaves the sign, the gate silu(1)
    out = plain.time_mixing(torch.ones(3, 1, dtype=torch.float64), t, "p.", {"heads": 1, "dim": 1}, 0.0)
    assert torch.allclose(out, float(plain.silu(f64(1.0))) * torch.ones(3, 1, dtype=torch.float64))
    # a shift of all positions changes no score: the rotation enters through position differences only
    q, k = torch.randn(4, 1, 6, dtype=torch.float64), torch.randn(4, 1, 6, dtype=torch.float64)
    turn = lambda x, shift: plain.rotate_pairs(x, torch.arange(4) + shift, 50.0, 4, torch.float64)[:, 0]
    assert torch.allclose(turn(q, 0) @ turn(k, 0).T, turn(q, 900) @ turn(k, 900).T, atol=1e-9)


# -- generation through the entry point, the scheduler and the engine ------------------------------------------------------
def test_greedy_generation_through_the_entry_point_equals_the_oracles():
    """More requests than places, prompts cut into portions by the token budget, a pool so small that requests wait
    for pages: the engine's own scheduler, cache manager, step function and sampler produce the oracle's tokens."""
    from llmserver_amd.entrypoints import generate
    for case, vocab in (("BA", 97), ("BB", 130)):
        raw, tensors = plain_model(case)
        prompts = [random_tokens(vocab, n, 700 + n) for n in (19, 3, 41, 8, 1, 27)]
        expected = [plain.greedy_generate(raw, tensors, prompt, 7) for prompt in prompts]
        got = generate(model_folder(case), prompts, max_new_tokens=7, dtype="float32", device="cpu", block_size=8, num_blocks=26,
                       max_batch_size=3, max_num_batched_tokens=24, prefill_chunk_size=16, ops=TorchOps())
        assert got == expected
